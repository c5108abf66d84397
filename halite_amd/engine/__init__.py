from .batch import Segment, StepContext
from .engine import InferenceEngine
from .runner import ModelRunner, StepError
from .scheduler import FinishReason, Request, Scheduler, SchedulerStats, StepPlan
from .types import InferenceRequest, InferenceResult

__all__ = [
    "FinishReason", "InferenceEngine", "InferenceRequest", "InferenceResult", "ModelRunner",
    "Request", "Scheduler", "SchedulerStats", "Segment", "StepContext", "StepError", "StepPlan",
]
