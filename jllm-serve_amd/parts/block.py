"""How the parts of one layer are arranged.

"prenorm" (model/LayerSpec.java:18-19; cpu/CpuBackend.java:959-969): xb = norm_in(x); x += mixer(xb);
xb = norm_post(x); x += ffn(xb). The residual stream x is fp32 and is never normalised itself.

Norms between two products need no launch of their own when both sides agree (optional, by attributes of the
parts; a part that knows nothing of this works as before):
* a mixer / feed-forward with ``takes_normed_rows = True`` only feeds its input to ``ops.gemm`` and so may get the
  norm as a promise (``norm.defer`` / ``ops.NormedRows``) instead of a tensor;
* one with ``prepares_next_norm = True`` takes ``then_norm=<norm part>`` in ``forward``, ends with
  ``then_norm.after_add(...)`` instead of the add into the residual, and returns that promise.
"""
from __future__ import annotations

from .base import Part, part_factory, register_part


class PreNormBlock(Part):
    def __init__(self, spec, prefix, build, positions):
        self.norm_in = part_factory("norm", spec.norm.kind)(spec.norm, build.hidden, f"{prefix}.{spec.norm_in_name}.weight", build)
        self.norm_post = part_factory("norm", spec.norm.kind)(spec.norm, build.hidden, f"{prefix}.{spec.norm_post_name}.weight",
                                                            build)
        self.mixer = part_factory("mixer", spec.mixer.kind)(spec.mixer, prefix, build, positions)
        self.ffn = part_factory("ffn", spec.ffn.kind)(spec.ffn, prefix, build)
        self.parts = (self.norm_in, self.mixer, self.norm_post, self.ffn)
        self.capturable = all(getattr(p, "capturable", True) for p in self.parts)

    def weight_specs(self):
        return [w for p in self.parts for w in p.weight_specs()]

    def load(self, get):
        for p in self.parts:
            p.load(get)

    def cache_spec(self):
        return self.mixer.cache_spec()

    def state_spec(self):
        return self.mixer.state_spec()

    def step_planners(self):
        return [pl for p in self.parts for pl in (p.step_planners() if hasattr(p, "step_planners") else [])]

    chains_norms = True  # forward takes normed_in / next_norm and returns the next block's input promise

    @staticmethod
    def _input(norm, consumer, x, promise):
        if getattr(consumer, "takes_normed_rows", False) and hasattr(norm, "defer"):
            if promise is not None and promise.x is x and promise.gain is getattr(norm, "gain", None):
                return promise
            return norm.defer(x)
        return norm.forward(x)

    def forward(self, x, step, slot, normed_in=None, next_norm=None):
        """``normed_in``: norm_in of x, prepared by whoever wrote x last (or None); ``next_norm``: the norm part that
        will read x next. Returns that norm of the new x as a promise when the feed-forward prepared it."""
        xb = self._input(self.norm_in, self.mixer, x, normed_in)
        if getattr(self.mixer, "prepares_next_norm", False) and hasattr(self.norm_post, "after_add"):
            mid = self.mixer.forward(xb, x, step, slot, then_norm=self.norm_post)
        else:
            self.mixer.forward(xb, x, step, slot)
            mid = None
        xb = self._input(self.norm_post, self.ffn, x, mid)
        if next_norm is not None and getattr(self.ffn, "prepares_next_norm", False) and hasattr(next_norm, "after_add"):
            return self.ffn.forward(xb, x, step, then_norm=next_norm)
        self.ffn.forward(xb, x, step)
        return None


register_part("arrangement", "prenorm", PreNormBlock, replace=True)
