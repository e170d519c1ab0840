"""The step function, the scheduler above it and the engine loop."""

from .batch import SeqChunk, StepContext
from .engine import Engine, StreamEvent
from .request import Request, RequestState, SamplingParams
from .scheduler import Plan, Scheduler, Work

__all__ = ["Engine", "Plan", "Request", "RequestState", "SamplingParams", "Scheduler",
           "SeqChunk", "StepContext", "StreamEvent", "Work"]
