"""One registry from an architecture's name (config.json `architectures[0]`) to its model.

The reference dispatches on the checkpoint's architecture tag by exact match and names the
implemented set when the tag is unknown (crates/beholdd-model/src/qwen3moe.rs:476-495).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

from .config.base import ConfigError, architecture_name


@dataclass(frozen=True)
class ArchitectureEntry:
    name: str
    config_class: type
    build: Callable       # build(config) -> model (no weights yet)


_ARCHITECTURES: dict = {}


def register_architecture(name: str, config_class: type, build: Callable) -> ArchitectureEntry:
    if name in _ARCHITECTURES:
        raise ValueError(f"architecture {name!r} is already registered")
    entry = ArchitectureEntry(name, config_class, build)
    _ARCHITECTURES[name] = entry
    return entry


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def resolve_architecture(config_dict: dict, origin: str = "config.json") -> ArchitectureEntry:
    name = architecture_name(config_dict, origin)
    entry = _ARCHITECTURES.get(name)
    if entry is None:
        raise ConfigError(f"{origin}: unsupported architecture {name!r}; implemented architectures are "
                          + ", ".join(registered_architectures()))
    return entry
