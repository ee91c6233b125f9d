"""Dense gated feed-forward: x += W_down (silu(W_gate xb) * (W_up xb)) (cpu/CpuBackend.java:661-669,
:1289-1300; tensors model/MlpWeights.java:19-33). The activation and product are the epilogue of the
gate/up product; the residual add is the epilogue of the down product."""
from __future__ import annotations

from ..config.schema import GatedMlpSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import BuildContext, Part, register_part


class GatedMlp(Part):
    takes_normed_rows = True    # the input goes into ops.gemm and nowhere else
    prepares_next_norm = True   # forward(then_norm=...) ends with then_norm.after_add and returns its promise
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

    def forward(self, xb, residual, step, then_norm=None):
        h = ops.gemm(xb, self.w_gate, w2=self.w_up, epilogue=ops.EPI_GATED, out_dtype=self.build.dtype,
                     exact=self.build.exact)
        if then_norm is not None:
            return then_norm.after_add(h, self.w_down, residual, exact=self.build.exact)
        ops.gemm(h, self.w_down, out=residual, epilogue=ops.EPI_ADD, exact=self.build.exact)
        return None


register_part("ffn", "gated_mlp", GatedMlp, replace=True)
