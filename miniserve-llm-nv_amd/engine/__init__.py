from .batch import StepEntry, build_step
from .engine import Engine, GenerationResult, StepOutput
from .plan import DecodeItem, ExecutionPlan, PrefillItem
from .request import Request, SamplingParams
from .runner import ModelRunner
from .scheduler import Scheduler
from .sequence import RequestStatus, SequenceState, SequenceView

__all__ = [
    "DecodeItem",
    "Engine",
    "ExecutionPlan",
    "GenerationResult",
    "ModelRunner",
    "PrefillItem",
    "Request",
    "RequestStatus",
    "SamplingParams",
    "Scheduler",
    "SequenceState",
    "SequenceView",
    "StepEntry",
    "StepOutput",
    "build_step",
]
