from .loader import WeightLoadError, WeightLoadReport, load_weights, weight_files
from .random_init import random_device_tensors, random_model_tensors, random_tensors, register_init, write_random_model

__all__ = [
    "WeightLoadError",
    "WeightLoadReport",
    "load_weights",
    "random_device_tensors",
    "random_model_tensors",
    "random_tensors",
    "register_init",
    "weight_files",
    "write_random_model",
]
