"""Strict readers for values of a ``config.json`` mapping.

Nothing is coerced: an integer key must hold a real ``int`` (not a bool, a
float or a string), a numeric key a real number, a boolean key a real ``bool``.
The same rule as the reference's ``ModelConfig.from_hf_config``
(reference: miniserve/config/model_config.py:73-107).
"""

from __future__ import annotations

import math
from typing import Any, Mapping

_MISSING = object()


class ConfigError(ValueError):
    """A ``config.json`` (or an engine option) that this framework does not run."""


def read_int(data: Mapping[str, Any], name: str, default: Any = _MISSING) -> int:
    value = data.get(name, default)
    if value is _MISSING or not isinstance(value, int) or isinstance(value, bool):
        raise ConfigError(f"{name} must be an integer in the model config.")
    return value


def read_positive_int(data: Mapping[str, Any], name: str, default: Any = _MISSING) -> int:
    value = read_int(data, name, default)
    if value <= 0:
        raise ConfigError(f"{name} must be positive.")
    return value


def read_number(data: Mapping[str, Any], name: str, default: Any = _MISSING) -> float:
    value = data.get(name, default)
    if value is _MISSING or not isinstance(value, (int, float)) or isinstance(value, bool):
        raise ConfigError(f"{name} must be numeric in the model config.")
    return float(value)


def read_finite_positive(data: Mapping[str, Any], name: str, default: Any = _MISSING) -> float:
    value = read_number(data, name, default)
    if not math.isfinite(value) or value <= 0:
        raise ConfigError(f"{name} must be finite and positive.")
    return value


def read_bool(data: Mapping[str, Any], name: str, default: Any = _MISSING) -> bool:
    value = data.get(name, default)
    if value is _MISSING or not isinstance(value, bool):
        raise ConfigError(f"{name} must be boolean in the model config.")
    return value


def read_str(data: Mapping[str, Any], name: str, default: Any = _MISSING) -> str:
    value = data.get(name, default)
    if value is _MISSING or not isinstance(value, str):
        raise ConfigError(f"{name} must be a string in the model config.")
    return value


def read_architecture(data: Mapping[str, Any]) -> str:
    """The single entry of ``architectures`` (reference: model_config.py:108-109)."""

    architectures = data.get("architectures")
    if (
        not isinstance(architectures, (list, tuple))
        or len(architectures) != 1
        or not isinstance(architectures[0], str)
    ):
        raise ConfigError("architectures must be a list with exactly one name.")
    return architectures[0]
