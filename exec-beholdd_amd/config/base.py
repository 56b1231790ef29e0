"""Typed reading of a checkpoint's config.json.

Every number a model uses comes from the file; a key that the formulas need and the file
does not give is an error, never a default.  The reference reads its hyperparameters the
same way from checkpoint metadata (crates/beholdd-model/src/qwen3moe.rs:157-180).
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass


class ConfigError(ValueError):
    """config.json is missing, malformed, or asks for something that is not implemented."""


@dataclass(frozen=True)
class LayerKinds:
    """Which parts one layer is made of; the model builder looks each name up in the part registries.

    Any configuration class can describe a decoder to `models.build_decoder` with
        layer_kinds() -> list[LayerKinds]      one per layer
        schedule()    -> list[(layer index, cache entry index)]
        vocab, hidden, max_position            the sizes the generic builder reads itself
        tie_word_embeddings                    optional, false when absent
    Everything else (head counts, widths, constants) is read only by the builders registered for the part
    names it uses, so a configuration with other field names registers builders of its own."""
    mixer: str
    feed_forward: str
    norm: str
    block: str


_MISSING = object()


class ConfigReader:
    """Checked access to the keys of one config.json dictionary."""

    def __init__(self, data: dict, origin: str = "config.json"):
        if not isinstance(data, dict):
            raise ConfigError(f"{origin}: top level must be a JSON object")
        self.data = data
        self.origin = origin

    def has(self, key: str) -> bool:
        return key in self.data and self.data[key] is not None

    def raw(self, key: str, default=_MISSING):
        if not self.has(key):
            if default is _MISSING:
                raise ConfigError(f"{self.origin}: required key {key!r} is missing")
            return default
        return self.data[key]

    # The kernels take their sizes as 32-bit integers: no size in a configuration may be larger.
    MOST = 2 ** 31 - 1

    def integer(self, key: str, default=_MISSING, minimum: int | None = None, maximum: int | None = MOST) -> int:
        value = self.raw(key, default)
        if isinstance(value, bool) or not isinstance(value, int):
            if isinstance(value, float) and value.is_integer():
                value = int(value)
            else:
                raise ConfigError(f"{self.origin}: {key!r} must be an integer, got {value!r}")
        if minimum is not None and value < minimum:
            raise ConfigError(f"{self.origin}: {key!r} must be at least {minimum}, got {value}")
        if maximum is not None and value > maximum:
            raise ConfigError(f"{self.origin}: {key!r} must be at most {maximum}, got {value}")
        return value

    def number(self, key: str, default=_MISSING) -> float:
        value = self.raw(key, default)
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"{self.origin}: {key!r} must be a number, got {value!r}")
        value = float(value)
        if not math.isfinite(value):
            raise ConfigError(f"{self.origin}: {key!r} must be finite, got {value}")
        return value

    def boolean(self, key: str, default=_MISSING) -> bool:
        value = self.raw(key, default)
        if not isinstance(value, bool):
            raise ConfigError(f"{self.origin}: {key!r} must be true or false, got {value!r}")
        return value

    def string(self, key: str, default=_MISSING) -> str:
        value = self.raw(key, default)
        if not isinstance(value, str):
            raise ConfigError(f"{self.origin}: {key!r} must be a string, got {value!r}")
        return value


def read_config_json(model_dir_or_file: str) -> tuple[dict, str]:
    """Return (dictionary, path) of a model folder's config.json or of a JSON file itself."""
    if not isinstance(model_dir_or_file, (str, os.PathLike)):
        # an integer would be taken for an open file's number by the calls below
        raise ConfigError(f"a model folder is named by a path, got {model_dir_or_file!r}")
    path = os.fspath(model_dir_or_file)
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as handle:
            data = json.load(handle)
    except FileNotFoundError:
        raise ConfigError(f"{path}: no such file") from None
    except json.JSONDecodeError as error:
        raise ConfigError(f"{path}: not valid JSON ({error})") from None
    if not isinstance(data, dict):
        raise ConfigError(f"{path}: top level must be a JSON object")
    return data, path


def architecture_name(data: dict, origin: str = "config.json") -> str:
    """The registry tag: `architectures[0]` of config.json."""
    names = data.get("architectures")
    if not isinstance(names, list) or len(names) != 1 or not isinstance(names[0], str):
        raise ConfigError(
            f"{origin}: 'architectures' must be a list with exactly one model class name, got {names!r}")
    return names[0]
