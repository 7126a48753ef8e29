from .engine import ContinuousBatchEngine, Engine
from .options import EngineOptions, parse_dtype
from .scheduler import ContinuousBatchScheduler, InferenceRequest, RequestState, ScheduledBatch
from .step import ModelRunner, StepEntry

__all__ = ["ContinuousBatchEngine", "Engine", "EngineOptions", "parse_dtype", "ContinuousBatchScheduler",
           "InferenceRequest", "RequestState", "ScheduledBatch", "ModelRunner", "StepEntry"]
