"""One registry from an architecture's name (``config.json``'s ``architectures[0]``) to its
typed configuration, and through it to its model.

The reference never reads ``architectures``: every entry point imports its one model class
directly (miniserve/server/__main__.py:16,74, bench/offline.py:50,396). Here the name picks the
configuration class; the configuration lowers itself to a ``ModelSpec`` from which the generic
model is assembled out of registered parts.
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Any, Protocol

from .spec import ModelSpec


class ArchitectureConfig(Protocol):
    """What a typed configuration must offer to be registered."""

    @classmethod
    def from_dict(cls, cfg: dict) -> "ArchitectureConfig": ...

    def to_spec(self) -> ModelSpec: ...

    def to_dict(self) -> dict: ...


ARCHITECTURES: dict[str, type] = {}


def register_architecture(name: str):
    """Class decorator: ``@register_architecture("Qwen3ForCausalLM")``."""

    def deco(cls):
        if name in ARCHITECTURES and ARCHITECTURES[name] is not cls:
            raise ValueError(f"architecture {name!r} is already registered")
        ARCHITECTURES[name] = cls
        cls.architecture = name
        return cls

    return deco


def unregister_architecture(name: str) -> None:
    ARCHITECTURES.pop(name, None)


def load_config_dict(path: str | Path) -> dict:
    """The raw ``config.json`` of a model folder (miniserve/model/weights.py:56-57)."""
    file = Path(path) / "config.json"
    if not file.is_file():
        raise FileNotFoundError(f"no config.json in {path}")
    return json.loads(file.read_text())


def architecture_name(cfg: dict) -> str:
    archs = cfg.get("architectures")
    if not archs or not isinstance(archs, (list, tuple)) or not isinstance(archs[0], str):
        raise ValueError(
            f"config.json names no architecture (key 'architectures'); known: {sorted(ARCHITECTURES)}"
        )
    return archs[0]


def config_from_dict(cfg: dict) -> Any:
    """The typed configuration the dictionary's architecture name selects."""
    name = architecture_name(cfg)
    try:
        cls = ARCHITECTURES[name]
    except KeyError:
        raise ValueError(f"unknown architecture {name!r}, expected one of {sorted(ARCHITECTURES)}") from None
    return cls.from_dict(cfg)


def load_config(path: str | Path) -> Any:
    return config_from_dict(load_config_dict(path))
