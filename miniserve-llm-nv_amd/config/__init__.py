from .engine_config import DTYPES, EngineConfig
from .fields import ConfigError
from .model_spec import LayerCall, LayerSpec, ModelSpec, PartSpec
from .registry import config_from_dict, load_config, register_architecture, registered_architectures
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
    "config_from_dict",
    "load_config",
    "register_architecture",
    "registered_architectures",
]
