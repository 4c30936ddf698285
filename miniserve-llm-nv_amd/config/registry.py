"""One registry from the architecture's name (``config.json: architectures[0]``)
to its configuration class.  The reference selects the family with an if/elif
on the same key (reference: miniserve/config/model_config.py:108-129,172-176)."""

from __future__ import annotations

import json
from pathlib import Path
from typing import Any, Mapping, Protocol

from .fields import ConfigError, read_architecture
from .model_spec import ModelSpec


class ArchitectureConfig(Protocol):
    """What an architecture's configuration class must offer."""

    architecture: str

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "ArchitectureConfig": ...

    def to_dict(self) -> dict[str, Any]: ...

    def model_spec(self) -> ModelSpec: ...


_ARCHITECTURES: dict[str, type] = {}


def register_architecture(name: str, config_class: type) -> None:
    if not isinstance(name, str) or not name:
        raise ValueError("architecture name must be a non-empty string.")
    for attribute in ("from_dict", "to_dict", "model_spec"):
        if not callable(getattr(config_class, attribute, None)):
            raise TypeError(f"{config_class!r} lacks {attribute}().")
    _ARCHITECTURES[name] = config_class


def registered_architectures() -> tuple[str, ...]:
    return tuple(sorted(_ARCHITECTURES))


def config_from_dict(data: Mapping[str, Any]) -> ArchitectureConfig:
    architecture = read_architecture(data)
    try:
        config_class = _ARCHITECTURES[architecture]
    except KeyError:
        raise ConfigError(
            f"UNSUPPORTED_MODEL_CONFIGURATION: architecture {architecture!r} is not registered "
            f"(registered: {', '.join(registered_architectures()) or 'none'})."
        ) from None
    return config_class.from_dict(data)


def load_config(model_dir: str | Path) -> ArchitectureConfig:
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"{path} does not exist.")
    data = json.loads(path.read_text(encoding="utf-8"))
    if not isinstance(data, dict):
        raise ConfigError("config.json must hold a JSON object.")
    return config_from_dict(data)


PRESET_DIR = Path(__file__).resolve().parent / "presets"


def preset_names() -> tuple[str, ...]:
    """Names of the ``config.json`` files that ship with the package: the layer sizes
    of served models, for runs with random weights."""

    return tuple(sorted(path.stem for path in PRESET_DIR.glob("*.json")))


def config_dict_from_preset_or_file(name_or_path: str) -> dict[str, Any]:
    """The ``config.json`` mapping of a preset (by name, any case) or of a file."""

    path = Path(name_or_path)
    if not path.is_file():
        path = PRESET_DIR / f"{name_or_path.lower()}.json"
        if not path.is_file():
            raise FileNotFoundError(
                f"{name_or_path!r} is neither a config.json nor one of the presets {', '.join(preset_names())}."
            )
    data = json.loads(path.read_text(encoding="utf-8"))
    if not isinstance(data, dict):
        raise ConfigError(f"{path} must hold a JSON object.")
    return data
