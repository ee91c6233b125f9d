"""Sampling parameters and the sampler."""
from .params import SamplingParams
from .sampler import SamplerState, sample_rows, select_rows, uniform

__all__ = ["SamplingParams", "SamplerState", "sample_rows", "select_rows", "uniform"]
