"""RMSNorm: y = (x * rsqrt(mean(x^2) + eps)) * g over fp32 rows (cpu/VectorKernels.java:630-634)."""
from __future__ import annotations

from ..config.schema import NormSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import BuildContext, Part, register_part


class RMSNorm(Part):
    def __init__(self, spec: NormSpec, dim: int, weight_name: str, build: BuildContext):
        self.eps = float(spec.eps)
        self.dim = dim
        self.weight_name = weight_name
        self.out_dtype = build.dtype
        self.gain = None

    def weight_specs(self):
        return [WeightSpec(self.weight_name, (self.dim,), init="gain")]

    def load(self, get):
        self.gain = get(self.weight_name)

    def forward(self, x, rows=None):
        return ops.rmsnorm(x, self.gain, self.eps, self.out_dtype, rows)


register_part("norm", "rmsnorm", RMSNorm, replace=True)
