"""Grouped-query attention over the paged cache.

The reference's step (cpu/CpuBackend.java:423-457, :543-583, :595-633): q, k, v projections (+ biases
right after the projection), per-head RMSNorm of q and k with gains shared by all heads, rotate-half RoPE
at each row's own position, store of k and v at those positions, causal attention of every row over its
own request's cache (query head h uses kv head h / G), then x += W_o att (+ b_o).

Here the three projections are one product with the stacked weight [q | k | v] (stacked at load from the
three named tensors); norm, rotation and the page write are one kernel; the residual add is the epilogue
of the output product.
"""
from __future__ import annotations

import torch

from ..cache.manager import KvSpec
from ..config.schema import GqaSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import BuildContext, Part, register_part


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
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = self.g_q = self.g_k = None

    def weight_specs(self):
        s, p, d = self.spec, self.prefix + ".self_attn.", self.build.hidden
        out = [WeightSpec(p + "q_proj.weight", (s.q_dim, d)), WeightSpec(p + "k_proj.weight", (s.kv_dim, d)),
               WeightSpec(p + "v_proj.weight", (s.kv_dim, d)), WeightSpec(p + "o_proj.weight", (d, s.q_dim))]
        if s.bias:
            out += [WeightSpec(p + "q_proj.bias", (s.q_dim,), init="bias"),
                    WeightSpec(p + "k_proj.bias", (s.kv_dim,), init="bias"),
                    WeightSpec(p + "v_proj.bias", (s.kv_dim,), init="bias")]
        if s.out_bias:
            out.append(WeightSpec(p + "o_proj.bias", (d,), init="bias"))
        if s.qk_norm:
            out += [WeightSpec(p + "q_norm.weight", (s.head_dim,), init="gain"),
                    WeightSpec(p + "k_norm.weight", (s.head_dim,), init="gain")]
        return out

    def load(self, get):
        s, p = self.spec, self.prefix + ".self_attn."
        parts = [get(p + f"{n}_proj.weight") for n in "qkv"]
        dt = parts[0].dtype if all(t.dtype == parts[0].dtype for t in parts) else torch.float32
        self.w_qkv = torch.cat([t.to(dt) for t in parts], dim=0).contiguous()
        del parts
        self.w_o = get(p + "o_proj.weight")
        if s.bias:
            self.b_qkv = torch.cat([get(p + f"{n}_proj.bias").to(torch.float32) for n in "qkv"]).contiguous()
        if s.out_bias:
            self.b_o = get(p + "o_proj.bias")
        if s.qk_norm:
            self.g_q = get(p + "q_norm.weight")
            self.g_k = get(p + "k_norm.weight")
            if self.g_q.dtype != self.g_k.dtype:
                self.g_q, self.g_k = self.g_q.float(), self.g_k.float()

    def cache_spec(self):
        return KvSpec(self.spec.kv_heads, self.spec.head_dim, self.spec.window)

    def forward(self, xb, residual, step, slot, then_norm=None):
        s = self.spec
        g = step.groups[slot.group]
        qkv = ops.gemm(xb, self.w_qkv, bias=self.b_qkv, out_dtype=self.build.dtype, exact=self.build.exact)
        rot = self.position.rotary() if self.position is not None else None
        cos, sin, rdim = rot if rot is not None else (None, None, 0)
        if not self.build.exact and step.meta is not None and step.meta.get("decode_only"):
            # single rows per request: norm, rotation and cache store happen inside the attention kernel
            att = ops.decode_attention_fused(qkv, slot.k_cache, slot.v_cache, g.block_table, step.row_req, step.positions,
                                             g.slots, cos, sin, self.g_q, self.g_k, s.qk_norm_eps, s.heads, s.kv_heads,
                                             s.head_dim, rdim, s.window, s.scale, step.meta, write_kv=slot.writes)
            if att is not None:
                return self._project_out(att, residual, then_norm)
        ops.qk_norm_rope_store(qkv, step.positions, g.slots, cos, sin, self.g_q, self.g_k, s.qk_norm_eps, s.heads,
                               s.kv_heads, s.head_dim, rdim, slot.k_cache.shape[2], slot.k_cache, slot.v_cache,
                               write_kv=slot.writes)
        att = ops.paged_attention(qkv[:, :s.q_dim], slot.k_cache, slot.v_cache, g.block_table, step.row_req,
                                  step.positions, s.heads, s.kv_heads, s.head_dim, s.window, s.scale, meta=step.meta,
                                  exact=self.build.exact)
        return self._project_out(att, residual, then_norm)

    def _project_out(self, att, residual, then_norm):
        if then_norm is not None:
            return then_norm.after_add(att, self.w_o, residual, bias=self.b_o, exact=self.build.exact)
        ops.gemm(att, self.w_o, bias=self.b_o, out=residual, epilogue=ops.EPI_ADD, exact=self.build.exact)
        return None


register_part("mixer", "gqa", GqaAttention, replace=True)
