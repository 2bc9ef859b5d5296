"""Strictly typed access to the members of a config.json object.

The reference reads every member with a whole-token parse and refuses wrong
types (src/model/huggingface.cpp:101-129); these readers do the same on a
parsed JSON object: an integer member must be a JSON integer (``true`` is not
one), a number must be finite, a boolean must be a literal.
"""
from __future__ import annotations

import json
import math
import os
from typing import Any, Mapping, Optional, Sequence

MAX_CONFIG_BYTES = 1 << 20  # src/model/huggingface.cpp:148


class ConfigError(ValueError):
    """A config.json that cannot be used: a missing key, a wrong type or a bad value."""


_MISSING = object()


def read_json_object(path: str) -> dict:
    size = os.path.getsize(path)
    if size == 0 or size > MAX_CONFIG_BYTES:
        raise ConfigError(f"{path}: config size {size} is invalid")
    with open(path, "r", encoding="utf-8") as handle:
        try:
            value = json.load(handle)
        except json.JSONDecodeError as error:
            raise ConfigError(f"{path}: not valid JSON: {error}") from None
    if not isinstance(value, dict):
        raise ConfigError(f"{path}: top level must be a JSON object")
    return value


def _get(source: Mapping[str, Any], key: str, default: Any):
    if key in source and source[key] is not None:
        return source[key]
    if default is _MISSING:
        raise ConfigError(f"config is missing {key}")
    return default


def integer(source: Mapping[str, Any], key: str, default: Any = _MISSING) -> Optional[int]:
    value = _get(source, key, default)
    if value is default and default is not _MISSING:
        return default
    if isinstance(value, bool) or not isinstance(value, int):
        raise ConfigError(f"config key {key} must be an integer, got {value!r}")
    return value


def number(source: Mapping[str, Any], key: str, default: Any = _MISSING) -> Optional[float]:
    value = _get(source, key, default)
    if value is default and default is not _MISSING:
        return default
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config key {key} must be a number, got {value!r}")
    value = float(value)
    if not math.isfinite(value):
        raise ConfigError(f"config key {key} must be finite")
    return value


def boolean(source: Mapping[str, Any], key: str, default: Any = _MISSING) -> Optional[bool]:
    value = _get(source, key, default)
    if value is default and default is not _MISSING:
        return default
    if not isinstance(value, bool):
        raise ConfigError(f"config key {key} must be true or false, got {value!r}")
    return value


def string(source: Mapping[str, Any], key: str, default: Any = _MISSING) -> Optional[str]:
    value = _get(source, key, default)
    if value is default and default is not _MISSING:
        return default
    if not isinstance(value, str):
        raise ConfigError(f"config key {key} must be a string, got {value!r}")
    return value


def string_list(source: Mapping[str, Any], key: str, default: Any = _MISSING) -> Optional[Sequence[str]]:
    value = _get(source, key, default)
    if value is default and default is not _MISSING:
        return default
    if not isinstance(value, list) or not all(isinstance(item, str) for item in value):
        raise ConfigError(f"config key {key} must be a list of strings, got {value!r}")
    return list(value)
