"""The decoder model assembled from parts: embedding, the layer schedule, final norm, output head.

Skeleton as cpu/CpuBackend.java:936-989 and :821-930: rows of all requests of a step form one activation
matrix; every layer runs over all rows; the final norm and the output head run only over the rows whose
logits are wanted (:895-912). The output head is the head tensor (``lm_head.weight`` for Qwen3) when the checkpoint
has it, else the embedding matrix (model/ModelWeights.java:36-43); the names come from the config's ``names``.

The order in which layers run is the config's ``schedule``: a list of runs, each naming a layer (a layer
may be named twice) and optionally an earlier run whose cache it reads instead of writing its own.
"""
from __future__ import annotations

from typing import List

import torch

from ..cache.manager import CacheEntryPlan
from ..config.schema import ModelConfig
from ..kernels import ops
from ..weights import loader
from ..weights.loader import WeightSpec
from .base import BuildContext, part_factory


class DecoderModel:
    def __init__(self, config: ModelConfig, dtype: torch.dtype, device, max_positions: int):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"the engine runs in float32 or bfloat16, not {dtype}")
        self.config = config
        self.dtype = dtype
        self.device = torch.device(device)
        self.build = BuildContext(hidden=config.hidden, dtype=dtype, device=self.device, max_positions=max_positions,
                                  exact=(dtype == torch.float32))
        self.positions = [part_factory("position", p.kind)(p, self.build) for p in config.positions]
        self.layers = [part_factory("arrangement", l.arrangement)(l, l.prefix, self.build, self.positions)
                       for l in config.layers]
        self.final_norm = part_factory("norm", config.final_norm.kind)(config.final_norm, config.hidden,
                                                                      config.names.final_norm, self.build)
        self.embed = None
        self.lm_head = None
        # a part that walks the step's requests on the host sets ``capturable = False``; then decode steps are
        # never recorded as graphs
        self.capturable = all(getattr(l, "capturable", True) for l in self.layers)

    # -------------------------------------------------------------------------------------------- weights

    def weight_specs(self) -> List[WeightSpec]:
        c = self.config
        specs = [WeightSpec(c.names.embed, (c.vocab, c.hidden))]
        for p in self.positions:  # a position encoding may have tensors of its own (a learned table)
            specs += p.weight_specs() if hasattr(p, "weight_specs") else []
        for l in self.layers:
            specs += l.weight_specs()
        specs += self.final_norm.weight_specs()
        specs.append(WeightSpec(c.names.head, (c.vocab, c.hidden), optional=c.tie_embeddings))
        return specs

    def load(self, source) -> None:
        loader.check(self.weight_specs(), source, where=self.config.description)

        def get(name):
            return loader.fetch(source, name, self.dtype, self.device)

        names = self.config.names
        self.embed = get(names.embed)
        for p in self.positions:
            if hasattr(p, "load"):
                p.load(get)
        for l in self.layers:
            l.load(get)
        self.final_norm.load(get)
        self.lm_head = get(names.head) if names.head in set(source.names()) else self.embed

    # -------------------------------------------------------------------------------------------- cache plan

    def cache_plans(self) -> List[CacheEntryPlan]:
        plans = []
        for e in self.config.schedule:
            layer = self.layers[e.layer]
            plans.append(CacheEntryPlan(kv=layer.cache_spec() if e.cache_from is None else None,
                                        cache_from=e.cache_from, state=layer.state_spec()))
        return plans

    def step_planners(self) -> list:
        """What the layers want to know about every batch (engine/step.py runs each distinct planner once per step)."""
        return [pl for l in self.layers for pl in (l.step_planners() if hasattr(l, "step_planners") else [])]

    # -------------------------------------------------------------------------------------------- forward

    def forward(self, step, slots) -> torch.Tensor:
        """Runs the step's rows through the schedule; returns fp32 logits [len(step.selected), vocab]."""
        x = ops.embed(self.embed, step.token_ids, self.config.embed_scale)
        for p in self.positions:  # an encoding that is added to the embedded rows rather than applied in the mixers
            if hasattr(p, "embed_add"):
                p.embed_add(x, step)
        schedule = self.config.schedule
        carry = None  # the next block's input norm, when the block before prepared it (parts/block.py)
        for run, e in enumerate(schedule):
            layer = self.layers[e.layer]
            if not getattr(layer, "chains_norms", False):
                layer.forward(x, step, slots[run])
                carry = None
                continue
            nxt = self.layers[schedule[run + 1].layer] if run + 1 < len(schedule) else None
            next_norm = getattr(nxt, "norm_in", None) if getattr(nxt, "chains_norms", False) else None
            carry = layer.forward(x, step, slots[run], normed_in=carry, next_norm=next_norm)
        if step.n_selected == 0:
            return torch.empty((0, self.config.vocab), dtype=torch.float32, device=self.device)
        xs = self.final_norm.forward(x, rows=step.selected)
        return ops.gemm(xs, self.lm_head, out_dtype=torch.float32, exact=self.build.exact)
