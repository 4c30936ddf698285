from .allocator import OutOfPagesError, PageAllocator
from .layout import CacheLayout, CallPlacement, KVGroup
from .manager import CacheError, CacheManager, CapacitySnapshot, SequenceStepMeta, StepItem, StepReservation
from .table import RETURNED, BlockTable

__all__ = [
    "BlockTable",
    "CacheError",
    "CacheLayout",
    "CacheManager",
    "CallPlacement",
    "CapacitySnapshot",
    "KVGroup",
    "OutOfPagesError",
    "PageAllocator",
    "RETURNED",
    "SequenceStepMeta",
    "StepItem",
    "StepReservation",
]
