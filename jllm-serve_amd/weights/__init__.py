"""Weights: the safetensors reader/writer, the by-name loader, the random-weights mode."""
from .safetensors_io import SafetensorsError, SafetensorsFile, SafetensorsSource, write_safetensors
from .loader import RandomSource, TensorSource, WeightError, WeightSpec, check, fetch, storage_dtype
from .random_init import write_random_model

__all__ = ["SafetensorsError", "SafetensorsFile", "SafetensorsSource", "write_safetensors", "RandomSource", "TensorSource",
           "WeightError", "WeightSpec", "check", "fetch", "storage_dtype", "write_random_model"]
