"""Registries from a part's kind to its class, one per category.

``register_part("mixer", "my_mixer", MyMixer)`` is all that is needed to make a
new kind usable from a ``ModelSpec``; nothing in the engine lists kinds.
"""
from __future__ import annotations

from typing import Callable, Dict

from .base import Part, Runtime
from .spec import PartSpec

_REGISTRIES: Dict[str, Dict[str, Callable[[PartSpec, Runtime], Part]]] = {}


def register_part(category: str, kind: str, factory: Callable[[PartSpec, Runtime], Part],
                  replace: bool = False) -> None:
    kinds = _REGISTRIES.setdefault(category, {})
    if kind in kinds and not replace:
        raise ValueError(f"{category} kind {kind!r} is already registered")
    kinds[kind] = factory


def unregister_part(category: str, kind: str) -> None:
    _REGISTRIES.get(category, {}).pop(kind, None)


def registered_kinds(category: str):
    return sorted(_REGISTRIES.get(category, {}))


def build_part(category: str, spec: PartSpec, runtime: Runtime) -> Part:
    kinds = _REGISTRIES.get(category, {})
    if spec.kind not in kinds:
        raise KeyError(f"unknown {category} kind {spec.kind!r}; registered: {', '.join(sorted(kinds)) or 'none'}")
    return kinds[spec.kind](spec, runtime)
