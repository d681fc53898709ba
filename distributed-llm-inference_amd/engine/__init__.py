"""Step function, scheduler and the engine's Python entry points."""

from .engine import LLMEngine, ModelRunner, RequestOutput, StepStats
from .request import FinishReason, Priority, Request, RequestStatus
from .scheduler import ScheduledChunk, Scheduler, SchedulerConfig, SchedulerOutput

__all__ = [
    "FinishReason", "LLMEngine", "ModelRunner", "Priority", "Request", "RequestOutput", "RequestStatus",
    "ScheduledChunk", "Scheduler", "SchedulerConfig", "SchedulerOutput", "StepStats",
]
