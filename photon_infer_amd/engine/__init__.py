from .options import EngineOptions, parse_dtype
from .step import ModelRunner, StepEntry

__all__ = ["EngineOptions", "parse_dtype", "ModelRunner", "StepEntry"]
