"""One registry from an architecture's name to its configuration class and model builder.

The reference has no registry, only a ``model_type`` string compare
(src/model/huggingface.cpp:153); here the name in config.json's
``architectures[0]`` chooses an ``Architecture``: how to read the typed
configuration, how to turn it into a ``ModelSpec`` and how to draw random weights.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, Mapping, Optional

from . import fields
from .fields import ConfigError


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[Mapping[str, Any]], Any]
    build_spec: Callable[[Any], Any]                      # configuration -> ModelSpec
    init_rules: Optional[Callable[[Any], Any]] = None     # configuration -> rules for random weights


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(architecture: Architecture, replace: bool = False) -> None:
    if architecture.name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {architecture.name!r} is already registered")
    _ARCHITECTURES[architecture.name] = architecture


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures():
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def _ensure_builtin() -> None:
    # Importing the module registers what the package itself provides.
    from .. import architectures  # noqa: F401


def architecture_named(name: str) -> Architecture:
    _ensure_builtin()
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unknown architecture {name!r}; registered: {', '.join(sorted(_ARCHITECTURES))}")
    return _ARCHITECTURES[name]


def architecture_of(source: Mapping[str, Any]) -> Architecture:
    names = fields.string_list(source, "architectures")
    if len(names) != 1:
        raise ConfigError(f"config key architectures must name exactly one architecture, got {names!r}")
    return architecture_named(names[0])


def load_config(folder_or_file: str):
    """Read config.json and return ``(architecture, typed configuration)``."""
    path = folder_or_file
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    source = fields.read_json_object(path)
    architecture = architecture_of(source)
    return architecture, architecture.config_from_dict(source)
