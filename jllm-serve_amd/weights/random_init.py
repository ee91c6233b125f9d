"""Random-weights mode: writes a model folder (config.json, model.safetensors) from a config and a seed.

The reference has no such mode in its engine; its tiny test checkpoints come from a script
(scripts/make-tiny-model.py:739-747, :801-822). The tensors written are exactly the ones the model's parts
declare, so a written folder always loads.
"""
from __future__ import annotations

import json
import os
from typing import Any, Mapping

import torch

from .loader import RandomSource
from .safetensors_io import write_safetensors


def model_weight_specs(config_dict: Mapping[str, Any]):
    """The configuration and the tensors its model asks for. The model class is the registry entry's, as everywhere:
    an architecture registered with a factory of its own gets its own tensor list."""
    from ..config import entry_for, parse_config
    from ..parts.model import DecoderModel
    cfg = parse_config(config_dict)
    factory = entry_for(cfg.model_type).model_factory or DecoderModel
    return cfg, factory(cfg, torch.bfloat16, "cpu", 1).weight_specs()


def random_source(config_dict: Mapping[str, Any], seed: int, std: float = 0.02, gain_std: float = 0.1,
                  dtype: torch.dtype = torch.bfloat16, device="cpu") -> RandomSource:
    _, specs = model_weight_specs(config_dict)
    return RandomSource(specs, seed, std=std, gain_std=gain_std, dtype=dtype, device=device)


def write_random_model(folder: str, config_dict: Mapping[str, Any], seed: int, std: float = 0.02,
                       gain_std: float = 0.1, dtype: torch.dtype = torch.bfloat16) -> str:
    """Matrices, embeddings and biases N(0, std); norm gains 1 + N(0, gain_std); values rounded to ``dtype``."""
    src = random_source(config_dict, seed, std, gain_std, dtype, "cpu")
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(dict(config_dict), f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"), {n: src.get(n) for n in src.names()},
                      metadata={"format": "pt", "seed": str(seed)})
    return folder
