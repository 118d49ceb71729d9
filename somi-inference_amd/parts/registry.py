"""Registries of part kinds: a plan names a part by (category, kind).

Adding a mixer, feed-forward, norm, position encoding or block arrangement is
one ``register_part`` call with a class of the matching interface; tests
register toy parts this way without touching the package.
"""

from __future__ import annotations

from typing import Any

from .base import PartSpec

CATEGORIES = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")
_PARTS: dict[str, dict[str, type]] = {c: {} for c in CATEGORIES}


def register_part(category: str, kind: str, cls: type, *, replace: bool = False) -> None:
    if category not in _PARTS:
        raise KeyError(f"unknown part category {category!r}; one of {CATEGORIES}")
    if kind in _PARTS[category] and not replace:
        raise KeyError(f"{category} kind {kind!r} is already registered")
    _PARTS[category][kind] = cls


def unregister_part(category: str, kind: str) -> None:
    _PARTS[category].pop(kind, None)


def part_kinds(category: str) -> list[str]:
    return sorted(_PARTS[category])


def build_part(category: str, spec: PartSpec, prefix: str, **extra: Any) -> Any:
    """Instantiate ``spec.kind`` of ``category`` with its params under ``prefix``."""
    kinds = _PARTS[category]
    if spec.kind not in kinds:
        raise KeyError(f"unknown {category} kind {spec.kind!r}; registered: {sorted(kinds)}")
    return kinds[spec.kind](prefix=prefix, **spec.params, **extra)
