"""How the parts of one layer are arranged.

"prenorm" (model/LayerSpec.java:18-19; cpu/CpuBackend.java:959-969): xb = norm_in(x); x += mixer(xb);
xb = norm_post(x); x += ffn(xb). The residual stream x is fp32 and is never normalised itself.
"""
from __future__ import annotations

from .base import Part, part_factory, register_part


class PreNormBlock(Part):
    def __init__(self, spec, prefix, build, positions):
        self.norm_in = part_factory("norm", spec.norm.kind)(spec.norm, build.hidden, prefix + ".input_layernorm.weight", build)
        self.norm_post = part_factory("norm", spec.norm.kind)(spec.norm, build.hidden,
                                                            prefix + ".post_attention_layernorm.weight", build)
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

    def forward(self, x, step, slot):
        xb = self.norm_in.forward(x)
        self.mixer.forward(xb, x, step, slot)
        xb = self.norm_post.forward(x)
        self.ffn.forward(xb, x, step)


register_part("arrangement", "prenorm", PreNormBlock, replace=True)
