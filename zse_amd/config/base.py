"""Typed configuration helpers and the architecture registry.

The reference registers one adapter per architecture under a short name and
detects it from ``architectures[]`` then ``model_type`` (format/arch/base.py:71-123).
Here the registry maps the architecture's own name (``architectures[0]``) to an
``Architecture``: its typed config class and the function that turns a config
into a ``ModelPlan``.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Callable, Dict, Iterable, Optional

from .plan import ModelPlan


class ConfigError(ValueError):
    """A config.json that cannot be served; the message names every problem found."""


@dataclass(frozen=True)
class Architecture:
    name: str                                   # e.g. "Gemma2ForCausalLM"
    config_from_dict: Callable[[dict], object]  # -> typed config (raises ConfigError)
    plan: Callable[[object], ModelPlan]
    model_types: tuple = ()                     # config.json "model_type" fallbacks


ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture) -> Architecture:
    ARCHITECTURES[arch.name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    ARCHITECTURES.pop(name, None)


def resolve_architecture(cfg: dict) -> Architecture:
    """Pick the architecture a config.json names.

    Exact match on ``architectures[*]`` first, then on ``model_type``
    (the reference's order, format/arch/base.py:91-123); an unknown name is an
    error that lists what is registered (format/arch/base.py:84-87).
    """
    for name in cfg.get("architectures") or []:
        if name in ARCHITECTURES:
            return ARCHITECTURES[name]
    mt = cfg.get("model_type")
    if mt:
        for arch in ARCHITECTURES.values():
            if mt in arch.model_types:
                return arch
    raise ConfigError(
        f"unknown architecture: architectures={cfg.get('architectures')!r}, "
        f"model_type={cfg.get('model_type')!r}; registered: {sorted(ARCHITECTURES)}")


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"no config.json in {model_dir}")
    with open(path, "r") as f:
        return json.load(f)


def load_config(model_dir: str):
    """(architecture, typed config) of a model folder."""
    raw = read_config_json(model_dir)
    arch = resolve_architecture(raw)
    return arch, arch.config_from_dict(raw)


class Problems:
    """Collects validation findings so that one error can list all of them."""

    def __init__(self, what: str):
        self.what = what
        self.items = []

    def add(self, msg: str) -> None:
        self.items.append(msg)

    def require(self, cond: bool, msg: str) -> None:
        if not cond:
            self.items.append(msg)

    def raise_if_any(self, exc=ConfigError) -> None:
        if self.items:
            raise exc(f"{self.what}: " + "; ".join(self.items))


def need(raw: dict, key: str, typ, problems: Problems, default=None, required=False,
         allow_none=False):
    """Read one key with a type check; a missing required key is recorded."""
    if key not in raw:
        if required:
            problems.add(f"missing required key '{key}'")
        return default
    v = raw[key]
    if v is None:
        if allow_none:
            return None
        if required:
            problems.add(f"required key '{key}' is null")
        return default
    if typ is float and isinstance(v, int) and not isinstance(v, bool):
        v = float(v)
    if (isinstance(v, bool) and typ is not bool) or not isinstance(v, typ):
        problems.add(f"key '{key}' must be {typ.__name__}, got {v!r}")
        return default
    return v
