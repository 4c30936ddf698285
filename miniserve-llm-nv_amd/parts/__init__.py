from .base import (
    CATEGORIES,
    GroupStepView,
    KVCacheNeed,
    KVCacheView,
    Part,
    StateNeed,
    StateView,
    StepContext,
    WeightSpec,
    build_block,
    build_part,
    register_part,
    registered_parts,
    unregister_part,
)
from . import attention, block, embedding, mlp, norm, rotary  # noqa: F401  (register the built-in parts)
from .model import CallCacheNeed, DecoderModel, TORCH_DTYPES

__all__ = [
    "CATEGORIES",
    "CallCacheNeed",
    "DecoderModel",
    "GroupStepView",
    "KVCacheNeed",
    "KVCacheView",
    "Part",
    "StateNeed",
    "StateView",
    "StepContext",
    "TORCH_DTYPES",
    "WeightSpec",
    "build_block",
    "build_part",
    "register_part",
    "registered_parts",
    "unregister_part",
]
