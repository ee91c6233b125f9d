"""The step function, the scheduler above it, and what builds them from a model folder."""
from .step import ModelRunner, StepContext, StepEntry, StepError
from .scheduler import Request, Scheduler, SchedulerConfig
from .engine import Engine, GenerationResult
from .build import build_model, build_runner, load_model, parse_dtype, require_gpu

__all__ = ["Engine", "GenerationResult", "Request", "Scheduler", "SchedulerConfig", "ModelRunner", "StepContext", "StepEntry", "StepError", "build_model", "build_runner", "load_model",
           "parse_dtype", "require_gpu"]
