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
        if spec.activation not in ops.GATE_FUNCTIONS:
            raise ValueError(f"unsupported activation '{spec.activation}': the product kernels have "
                             f"{sorted(ops.GATE_FUNCTIONS)} as gate functions")
        self.gate = ops.GATE_FUNCTIONS[spec.activation]
        self.hidden = spec.hidden
        self.names = spec.names
        self.dim = build.hidden
        self.prefix = prefix
        self.build = build
        self.w_gate = self.w_up = self.w_down = None

    def _name(self, which: str) -> str:
        return f"{self.prefix}.{getattr(self.names, which)}.weight"

    def weight_specs(self):
        if self.names.gate_up is not None:  # one stacked tensor [gate | up]
            return [WeightSpec(self._name("gate_up"), (2 * self.hidden, self.dim)),
                    WeightSpec(self._name("down"), (self.dim, self.hidden))]
        return [WeightSpec(self._name("gate"), (self.hidden, self.dim)), WeightSpec(self._name("up"), (self.hidden, self.dim)),
                WeightSpec(self._name("down"), (self.dim, self.hidden))]

    def load(self, get):
        if self.names.gate_up is not None:
            both = get(self._name("gate_up"))
            self.w_gate, self.w_up = both[:self.hidden], both[self.hidden:]  # contiguous halves of one tensor
        else:
            self.w_gate = get(self._name("gate"))
            self.w_up = get(self._name("up"))
        self.w_down = get(self._name("down"))

    def forward(self, xb, residual, step, then_norm=None):
        h = ops.gemm(xb, self.w_gate, w2=self.w_up, epilogue=ops.EPI_GATED, out_dtype=self.build.dtype,
                     exact=self.build.exact, gate=self.gate)
        if then_norm is not None:
            return then_norm.after_add(h, self.w_down, residual, exact=self.build.exact)
        ops.gemm(h, self.w_down, out=residual, epilogue=ops.EPI_ADD, exact=self.build.exact)
        return None


register_part("ffn", "gated_mlp", GatedMlp, replace=True)
