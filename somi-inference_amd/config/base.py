"""Typed reading of a model's ``config.json``.

The reference has no configuration type: it reads attributes of a library
object ad hoc (somi_inference/models/qwen2_adapter.py:205-225) and asserts
integers out of a dict (somi_inference/entrypoints/llm.py:49-52, 93-96).  Here
every architecture declares a frozen dataclass, built by a ``from_dict`` that
reads the architecture's own config.json keys through :class:`KeyReader`, so a
missing key, a wrong type and a violated rule each raise :class:`ConfigError`
with the key's name.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, ClassVar


class ConfigError(ValueError):
    """A config.json key is missing, has the wrong type or breaks a rule."""


_MISSING = object()


class KeyReader:
    """Reads typed values out of a parsed config.json and names what is wrong."""

    def __init__(self, data: dict[str, Any], where: str = "config.json") -> None:
        if not isinstance(data, dict):
            raise ConfigError(f"{where}: expected a JSON object, got {type(data).__name__}")
        self._data = data
        self._where = where

    def has(self, key: str) -> bool:
        return key in self._data and self._data[key] is not None

    def raw(self, key: str, default: Any = _MISSING) -> Any:
        if key in self._data and self._data[key] is not None:
            return self._data[key]
        if default is _MISSING:
            raise ConfigError(f"{self._where}: required key '{key}' is missing")
        return default

    def integer(self, key: str, default: Any = _MISSING, *, minimum: int | None = None) -> int:
        value = self.raw(key, default)
        if isinstance(value, bool) or not isinstance(value, int):
            raise ConfigError(f"{self._where}: '{key}' must be an integer, got {value!r}")
        if minimum is not None and value < minimum:
            raise ConfigError(f"{self._where}: '{key}' must be >= {minimum}, got {value}")
        return value

    def optional_integer(self, key: str, *, minimum: int | None = None) -> int | None:
        if not self.has(key):
            return None
        return self.integer(key, minimum=minimum)

    def number(self, key: str, default: Any = _MISSING, *, positive: bool = False) -> float:
        value = self.raw(key, default)
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"{self._where}: '{key}' must be a number, got {value!r}")
        value = float(value)
        if positive and not value > 0.0:
            raise ConfigError(f"{self._where}: '{key}' must be > 0, got {value}")
        return value

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        value = self.raw(key, default)
        if not isinstance(value, bool):
            raise ConfigError(f"{self._where}: '{key}' must be true or false, got {value!r}")
        return value

    def string(self, key: str, default: Any = _MISSING) -> str:
        value = self.raw(key, default)
        if not isinstance(value, str):
            raise ConfigError(f"{self._where}: '{key}' must be a string, got {value!r}")
        return value

    def sub(self, key: str) -> "KeyReader | None":
        if not self.has(key):
            return None
        value = self._data[key]
        if not isinstance(value, dict):
            raise ConfigError(f"{self._where}: '{key}' must be an object, got {value!r}")
        return KeyReader(value, f"{self._where}:{key}")


@dataclass(frozen=True)
class ModelConfig:
    """Base of every architecture's typed configuration.

    A subclass names the architecture string it answers to, lists its fields,
    and implements ``from_dict`` / ``to_dict`` over the architecture's own
    config.json keys.  ``to_dict`` must round-trip through ``from_dict``: the
    random-weights mode writes it as the model folder's config.json.
    """

    architecture: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, data: dict[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> dict[str, Any]:
        raise NotImplementedError


def read_config_json(model_dir: str | os.PathLike) -> dict[str, Any]:
    """Parse ``<model_dir>/config.json``; errors name the file."""
    path = os.path.join(os.fspath(model_dir), "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path}: no such file (a model folder holds config.json and model.safetensors)")
    with open(path, "r", encoding="utf-8") as handle:
        try:
            data = json.load(handle)
        except json.JSONDecodeError as err:
            raise ConfigError(f"{path}: not valid JSON ({err})") from err
    if not isinstance(data, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return data


def architecture_of(data: dict[str, Any]) -> str:
    """The architecture string of a parsed config.json (``architectures[0]``).

    The reference dispatches on ``model_type`` (somi_inference/models/loader.py:22);
    the class name in ``architectures`` is the finer key and is what a model
    folder written by any exporter carries, so it is the registry's key here.
    """
    archs = data.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json: 'architectures' must be a non-empty list of strings")
    return archs[0]
