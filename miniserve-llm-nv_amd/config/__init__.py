from .engine_config import DTYPES, EngineConfig
from .fields import ConfigError
from .model_spec import LayerCall, LayerSpec, ModelSpec, PartSpec
from .registry import (
    config_dict_from_preset_or_file,
    config_from_dict,
    load_config,
    preset_names,
    register_architecture,
    registered_architectures,
)
from .qwen3 import Qwen3Config

__all__ = [
    "ConfigError",
    "DTYPES",
    "EngineConfig",
    "LayerCall",
    "LayerSpec",
    "ModelSpec",
    "PartSpec",
    "Qwen3Config",
    "config_dict_from_preset_or_file",
    "config_from_dict",
    "load_config",
    "preset_names",
    "register_architecture",
    "registered_architectures",
]
