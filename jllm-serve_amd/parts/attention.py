"""Grouped-query attention over the paged cache.

The reference's step (cpu/CpuBackend.java:423-457, :543-583, :595-633): q, k, v projections (+ biases
right after the projection), per-head RMSNorm of q and k with gains shared by all heads, rotate-half RoPE
at each row's own position, store of k and v at those positions, causal attention of every row over its
own request's cache (query head h uses kv head h / G), then x += W_o att (+ b_o).

Here the three projections are one product with the stacked weight [q | k | v] (stacked at load from the
three tensors the spec names, or read as one tensor where the spec names a stacked one); norm, rotation and the page write are one kernel; the residual add is the epilogue
of the output product.
"""
from __future__ import annotations

import torch

from ..cache.manager import KvSpec
from ..config.schema import GqaSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import BuildContext, Part, register_part


TILE_ROWS = 128  # rows of one request that the portion-attention kernel takes per workgroup
# The portion kernel's two-group form pays when the run with the most keys has this many times the average (measured
# at 32 heads: 2,048 rows from position 0, ratio 1.9: 85 -> 70 us; from position 2,048, ratio 1.3: 174 / 170; from
# position 6,144, ratio 1.1: 334 -> 364, the one-group form is the faster one there)
UNEVEN_RUNS = 1.5


class GqaStepPlanner:
    """What the attention kernels want to know about a batch, made once per step for all attention layers: the
    portions cut into runs of at most TILE_ROWS rows, as (request, first row, rows, first position), the runs with
    the most keys first (their workgroups take longest and should start first); whether every request brings a
    single row (then the split-key kernels take the step); and, in a mixed step, whether the requests that bring a
    single row lie together (then those rows go through the kernel for single rows and the tile list ends before
    them); and whether the portions' runs differ much in their number of keys (one prompt from its start: the last
    run sees 16 times the keys of the first), which is when the portion kernel does well to cut every run's keys over
    two groups of waves."""

    key = ("gqa", TILE_ROWS)

    def plan(self, batch):
        from ..engine.step import StepPlan
        segments = batch.segments
        decode_only = all(s.n == 1 for s in segments)
        tiles = []
        n_multi = 0
        single_rows = None
        key_groups = 1
        if not decode_only:
            runs = [(s.index, s.row0 + r, min(TILE_ROWS, s.n - r), s.pos0 + r) for s in segments if s.n > 1
                    for r in range(0, s.n, TILE_ROWS)]
            runs.sort(key=lambda t: -(t[3] + t[2]))
            n_multi = len(runs)
            keys = [t[3] + t[2] for t in runs]
            if keys and max(keys) * len(keys) >= UNEVEN_RUNS * sum(keys):
                key_groups = 2
            ones = sorted(s.row0 for s in segments if s.n == 1)
            if ones and ones[-1] - ones[0] + 1 == len(ones):
                single_rows = (ones[0], len(ones))
            runs += [(s.index, s.row0, 1, s.pos0) for s in segments if s.n == 1]
            tiles = [v for t in runs for v in t]
        return StepPlan({"tiles": tiles}, {"decode_only": decode_only, "n_tiles": len(tiles) // 4,
                                           "n_tiles_multi": n_multi, "single_rows": single_rows,
                                           "key_groups": key_groups})


class GqaAttention(Part):
    takes_normed_rows = True    # the input goes into ops.gemm and nowhere else
    prepares_next_norm = True   # forward(then_norm=...) ends with then_norm.after_add and returns its promise
    def __init__(self, spec: GqaSpec, prefix: str, build: BuildContext, positions):
        if spec.kv_heads <= 0 or spec.heads % spec.kv_heads != 0:
            raise ValueError(f"{spec.kv_heads} kv heads do not divide {spec.heads} query heads")
        self.spec = spec
        self.prefix = prefix
        self.build = build
        self.position = positions[spec.position] if spec.position is not None else None
        rot = self.position.rotary() if self.position is not None else None
        try:  # sizes that no kernel takes are refused here, when the model is built, not at the first step
            ops.check_attention_shape(spec.heads, spec.kv_heads, spec.head_dim, rot[2] if rot is not None else 0)
        except ops.KernelError as e:
            raise ValueError(f"{prefix}: {e}") from None
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = self.g_q = self.g_k = None

    def _name(self, which: str, ending: str = ".weight") -> str:
        return f"{self.prefix}.{getattr(self.spec.names, which)}{ending}"

    def weight_specs(self):
        s, d, nm = self.spec, self.build.hidden, self.spec.names
        if nm.qkv is not None:  # one stacked tensor [q | k | v]
            out = [WeightSpec(self._name("qkv"), (s.q_dim + 2 * s.kv_dim, d))]
            if s.bias:
                out.append(WeightSpec(self._name("qkv", ".bias"), (s.q_dim + 2 * s.kv_dim,), init="bias"))
        else:
            out = [WeightSpec(self._name("q"), (s.q_dim, d)), WeightSpec(self._name("k"), (s.kv_dim, d)),
                   WeightSpec(self._name("v"), (s.kv_dim, d))]
            if s.bias:
                out += [WeightSpec(self._name("q", ".bias"), (s.q_dim,), init="bias"),
                        WeightSpec(self._name("k", ".bias"), (s.kv_dim,), init="bias"),
                        WeightSpec(self._name("v", ".bias"), (s.kv_dim,), init="bias")]
        out.append(WeightSpec(self._name("o"), (d, s.q_dim)))
        if s.out_bias:
            out.append(WeightSpec(self._name("o", ".bias"), (d,), init="bias"))
        if s.qk_norm:
            out += [WeightSpec(self._name("q_norm"), (s.head_dim,), init="gain"),
                    WeightSpec(self._name("k_norm"), (s.head_dim,), init="gain")]
        return out

    def load(self, get):
        s, nm = self.spec, self.spec.names
        if nm.qkv is not None:
            self.w_qkv = get(self._name("qkv"))
            if s.bias:
                self.b_qkv = get(self._name("qkv", ".bias")).to(torch.float32).contiguous()
        else:
            parts = [get(self._name(n)) for n in "qkv"]
            dt = parts[0].dtype if all(t.dtype == parts[0].dtype for t in parts) else torch.float32
            self.w_qkv = torch.cat([t.to(dt) for t in parts], dim=0).contiguous()
            del parts
            if s.bias:
                self.b_qkv = torch.cat([get(self._name(n, ".bias")).to(torch.float32) for n in "qkv"]).contiguous()
        self.w_o = get(self._name("o"))
        if s.out_bias:
            self.b_o = get(self._name("o", ".bias"))
        if s.qk_norm:
            self.g_q = get(self._name("q_norm"))
            self.g_k = get(self._name("k_norm"))
            if self.g_q.dtype != self.g_k.dtype:
                self.g_q, self.g_k = self.g_q.float(), self.g_k.float()

    def cache_spec(self):
        return KvSpec(self.spec.kv_heads, self.spec.head_dim, self.spec.window)

    def step_planners(self):
        return [GqaStepPlanner()]

    @staticmethod
    def _batch_facts(step):
        """The kernels' view of the batch: the step's own numbers and this mixer's plan of it."""
        plan = step.plans.get(GqaStepPlanner.key)
        meta = {"max_context": step.max_context, "requests": step.n_requests, "rows": step.n_tokens}
        if plan is None:  # a step put together without the planner: the general kernels take it
            meta["decode_only"] = False
            return meta
        meta.update(plan.facts)
        tiles = plan.arrays.get("tiles")
        meta["segments_dev"] = tiles if tiles is not None and tiles.numel() else None
        return meta

    def forward(self, xb, residual, step, slot, then_norm=None):
        s = self.spec
        g = step.groups[slot.group]
        k_cache, v_cache = slot.rows["k"], slot.rows["v"]
        meta = self._batch_facts(step)
        qkv = ops.gemm(xb, self.w_qkv, bias=self.b_qkv, out_dtype=self.build.dtype, exact=self.build.exact)
        rot = self.position.rotary() if self.position is not None else None
        cos, sin, rdim = rot if rot is not None else (None, None, 0)
        bias = getattr(self.position, "score_bias", None)
        slopes = bias(s.heads) if bias is not None else None  # an encoding that biases scores by distance
        if not self.build.exact and slopes is None and meta.get("decode_only"):
            # single rows per request: norm, rotation and cache store happen inside the attention kernel
            att = ops.decode_attention_fused(qkv, k_cache, v_cache, g.block_table, step.row_req, step.positions,
                                             g.slots, cos, sin, self.g_q, self.g_k, s.qk_norm_eps, s.heads, s.kv_heads,
                                             s.head_dim, rdim, s.window, s.scale, meta, write_kv=slot.writes)
            if att is not None:
                return self._project_out(att, residual, then_norm)
        ops.qk_norm_rope_store(qkv, step.positions, g.slots, cos, sin, self.g_q, self.g_k, s.qk_norm_eps, s.heads,
                               s.kv_heads, s.head_dim, rdim, slot.page_size, k_cache, v_cache, write_kv=slot.writes)
        att = ops.paged_attention(qkv[:, :s.q_dim], k_cache, v_cache, g.block_table, step.row_req,
                                  step.positions, s.heads, s.kv_heads, s.head_dim, s.window, s.scale, meta=meta,
                                  exact=self.build.exact, slopes=slopes)
        return self._project_out(att, residual, then_norm)

    def _project_out(self, att, residual, then_norm):
        if then_norm is not None:
            return then_norm.after_add(att, self.w_o, residual, bias=self.b_o, exact=self.build.exact)
        ops.gemm(att, self.w_o, bias=self.b_o, out=residual, epilogue=ops.EPI_ADD, exact=self.build.exact)
        return None


register_part("mixer", "gqa", GqaAttention, replace=True)
