"""One registry from an architecture's name to its configuration type and model plan.

The reference keeps ``MODEL_LOADERS = {"qwen2": load_from_hf}`` keyed by
``model_type`` and raises ``ValueError("Unsupported model type: X")`` on a miss
(somi_inference/models/loader.py:14-26).  Here the key is the class name in
config.json's ``architectures`` and the value holds two things: the typed
configuration class, and a function from that configuration to a
:class:`~somi_inference_amd.models.plan.ModelPlan` (pure data that names the
parts of every layer).  Nothing else in the package mentions an architecture by
name.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable

from .base import ConfigError, ModelConfig, architecture_of


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type[ModelConfig]
    build_plan: Callable[[Any], Any]   # (config) -> ModelPlan


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_class: type[ModelConfig],
                          build_plan: Callable[[Any], Any], *, replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ConfigError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_class, build_plan)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def resolve_architecture(name: str) -> Architecture:
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"Unsupported architecture: {name!r}; registered: {registered_architectures()}")
    return _ARCHITECTURES[name]


def config_from_dict(data: dict[str, Any]) -> tuple[Architecture, ModelConfig]:
    """Pick the architecture named by a parsed config.json and build its typed config."""
    arch = resolve_architecture(architecture_of(data))
    return arch, arch.config_class.from_dict(data)
