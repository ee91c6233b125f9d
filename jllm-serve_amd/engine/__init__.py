"""The step function, the scheduler above it, and what builds them from a model folder."""
from .step import ModelRunner, StepContext, StepEntry, StepError
from .build import build_model, build_runner, load_model, parse_dtype, require_gpu

__all__ = ["ModelRunner", "StepContext", "StepEntry", "StepError", "build_model", "build_runner", "load_model",
           "parse_dtype", "require_gpu"]
