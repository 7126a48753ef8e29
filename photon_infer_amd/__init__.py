"""photon_infer_amd: a small, whole LLM inference engine for one AMD MI355X GPU."""
from .errors import (CacheError, ConfigError, ErrorCode, KernelError, KernelLibraryMissing, OutOfMemoryError, OutOfPagesError,
                     PhotonError, RequestError, UnsupportedModelError, WeightError)
from .registry import (build_model_spec, get_architecture, load_config, register_architecture,
                       registered_architectures)

from .engine import ContinuousBatchEngine, Engine, EngineOptions, ModelRunner, StepEntry
from .sampling import SamplingParams
from .weights import write_random_model

__version__ = "0.1.0"

__all__ = [
    "ContinuousBatchEngine", "Engine", "EngineOptions", "ModelRunner", "StepEntry", "SamplingParams",
    "write_random_model",
    "CacheError", "ConfigError", "ErrorCode", "KernelError", "KernelLibraryMissing", "OutOfMemoryError", "OutOfPagesError",
    "PhotonError", "RequestError", "UnsupportedModelError", "WeightError", "build_model_spec",
    "get_architecture", "load_config", "register_architecture", "registered_architectures",
]
