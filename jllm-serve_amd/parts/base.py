"""Registries of the parts a layer is put together from, and the interfaces they keep.

The reference resolves a ``LayerPlan(weights, attention, residual, ffn)`` once per layer from the layer's
spec (cpu/CpuBackend.java:336-394); the sealed variants of its specs are where other layer kinds enter
(model/Attention.java:4, model/Mlp.java:4). Here each slot of a layer has a registry from the spec's
``kind`` to a class:

* ``position``  (spec, build) -> object with ``rotary() -> (cos, sin, rotary_dim) | None`` (rotation of q and k in
  the mixer); optionally ``score_bias(heads) -> fp32 [heads] | None`` (the attention adds slope * (key position -
  query position) to its scores) and ``embed_add(x, step)`` (the model calls it once on the embedded fp32 rows,
  for encodings that are added at the input); its own ``weight_specs()`` / ``load(get)`` are honoured
* ``norm``      (spec, dim, weight_name, build) -> ``forward(x_fp32, rows=None) -> activations``
* ``mixer``     (spec, prefix, build, positions) -> ``forward(xb, residual, step, slot)``; adds into residual
* ``ffn``       (spec, prefix, build) -> ``forward(xb, residual, step)``; adds into residual
* ``arrangement`` (layer spec, parts) -> ``forward(residual, step, slot)``

Every part also has ``weight_specs() -> [WeightSpec]`` and ``load(get)`` where ``get(name)`` returns the
tensor on the device in its storage type. A mixer may declare ``cache_spec() -> PageSpec | None`` (named
per-position tensors in pages), ``state_spec() -> StateSpec | None`` (fixed-size per-request state) and
``step_planners()`` (what it wants to know about every batch). No part knows which model it is in.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List

import torch

from ..weights.loader import WeightSpec

SLOTS = ("position", "norm", "mixer", "ffn", "arrangement")
_PARTS: Dict[str, Dict[str, Callable[..., Any]]] = {s: {} for s in SLOTS}


def register_part(slot: str, kind: str, factory: Callable[..., Any], replace: bool = False) -> None:
    if slot not in _PARTS:
        raise ValueError(f"unknown part slot '{slot}' (slots: {', '.join(SLOTS)})")
    if kind in _PARTS[slot] and not replace:
        raise ValueError(f"{slot} part '{kind}' is already registered")
    _PARTS[slot][kind] = factory


def unregister_part(slot: str, kind: str) -> None:
    _PARTS[slot].pop(kind, None)


def part_factory(slot: str, kind: str) -> Callable[..., Any]:
    try:
        return _PARTS[slot][kind]
    except KeyError:
        raise ValueError(f"no {slot} part of kind '{kind}' is registered (have: {sorted(_PARTS[slot])})") from None


@dataclass
class BuildContext:
    """What a part may know about the run it is built for."""

    hidden: int
    dtype: torch.dtype  # activations and cache: torch.float32 or torch.bfloat16
    device: torch.device
    max_positions: int  # longest sequence the engine will hold
    exact: bool = False  # float32 runs: plain-FMA kernels only


class Part:
    def weight_specs(self) -> List[WeightSpec]:
        return []

    def load(self, get) -> None:
        pass

    def cache_spec(self):
        return None

    def state_spec(self):
        return None

    def step_planners(self):
        """Planners for what this part wants to know about every batch beyond the step's own arrays: objects with
        ``key`` (equal keys plan once per step) and ``plan(StepBatch) -> StepPlan`` (engine/step.py); the part finds
        the result in ``step.plans[key]``."""
        return []
