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

    def defer(self, x):
        """The normalised rows as a promise, for consumers that feed them to ``ops.gemm`` only."""
        return ops.NormedRows(x, self.gain, self.eps, self.out_dtype)

    def after_add(self, a, w, residual, bias=None, exact=False):
        """residual += a @ w.T (+ bias), and this norm of the result as a promise: the product that makes the new
        residual rows can prepare their norm on its way out (``ops.gemm_add_then_norm``)."""
        return ops.gemm_add_then_norm(a, w, residual, self.gain, self.eps, self.out_dtype, bias=bias, exact=exact)


register_part("norm", "rmsnorm", RMSNorm, replace=True)
