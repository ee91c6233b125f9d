"""Dense gated feed-forward: x += W_down (silu(W_gate xb) * (W_up xb)) (cpu/CpuBackend.java:661-669,
:1289-1300; tensors model/MlpWeights.java:19-33). The activation and product are the epilogue of the
gate/up product; the residual add is the epilogue of the down product."""
from __future__ import annotations

from ..config.schema import GatedMlpSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import BuildContext, Part, register_part


class GatedMlp(Part):
    def __init__(self, spec: GatedMlpSpec, prefix: str, build: BuildContext):
        if spec.activation != "silu":
            raise ValueError(f"unsupported activation '{spec.activation}': only silu is built")
        self.hidden = spec.hidden
        self.dim = build.hidden
        self.prefix = prefix
        self.build = build
        self.w_gate = self.w_up = self.w_down = None

    def weight_specs(self):
        p = self.prefix + ".mlp."
        return [WeightSpec(p + "gate_proj.weight", (self.hidden, self.dim)),
                WeightSpec(p + "up_proj.weight", (self.hidden, self.dim)),
                WeightSpec(p + "down_proj.weight", (self.dim, self.hidden))]

    def load(self, get):
        p = self.prefix + ".mlp."
        self.w_gate = get(p + "gate_proj.weight")
        self.w_up = get(p + "up_proj.weight")
        self.w_down = get(p + "down_proj.weight")

    def forward(self, xb, residual, step):
        h = ops.gemm(xb, self.w_gate, w2=self.w_up, epilogue=ops.EPI_GATED, out_dtype=self.build.dtype,
                     exact=self.build.exact)
        ops.gemm(h, self.w_down, out=residual, epilogue=ops.EPI_ADD, exact=self.build.exact)


register_part("ffn", "gated_mlp", GatedMlp, replace=True)
