"""The step function, the scheduler above it and the engine loop.

Requests, sampling parameters, the scheduler, its plans and the per-step records are the host
core's (C++: ``csrc/host/scheduler.*``, ``engine_core.*``); they are named here for Python.
"""

from ..hostcore import core as _core
from .batch import SeqChunk, StepContext
from .engine import Engine

Plan = _core.Plan
Request = _core.Request
RequestState = _core.RequestState
SamplingParams = _core.SamplingParams
Scheduler = _core.Scheduler
StepRecord = _core.StepRecord
StreamEvent = _core.StreamEvent
Work = _core.Work

__all__ = ["Engine", "Plan", "Request", "RequestState", "SamplingParams", "Scheduler",
           "SeqChunk", "StepContext", "StepRecord", "StreamEvent", "Work"]
