"""Sampling parameters and the sampler."""
from .params import SamplingParams
from .sampler import SamplerState, sample_rows, uniform

__all__ = ["SamplingParams", "SamplerState", "sample_rows", "uniform"]
