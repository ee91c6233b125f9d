"""One registry from an architecture's name to its config parser and its model class.

The reference keeps a map model_type -> architecture class and one small parser per family
(model/Families.java:28-50, :107-128). Here an entry holds the parser (config.json dict -> ModelConfig)
and, optionally, a model factory; without one the generic decoder model assembled from registered
parts is used.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, Mapping, Optional

from .schema import ConfigError, ModelConfig


@dataclass(frozen=True)
class ArchitectureEntry:
    model_type: str
    architecture: str
    parse: Callable[[Mapping[str, Any], str, str], ModelConfig]
    model_factory: Optional[Callable[..., Any]] = None


_REGISTRY: Dict[str, ArchitectureEntry] = {}


def register_architecture(model_type: str, architecture: str, parse, model_factory=None, replace: bool = False) -> None:
    if model_type in _REGISTRY and not replace:
        raise ValueError(f"architecture '{model_type}' is already registered")
    _REGISTRY[model_type] = ArchitectureEntry(model_type, architecture, parse, model_factory)


def unregister_architecture(model_type: str) -> None:
    _REGISTRY.pop(model_type, None)


def supported() -> Dict[str, str]:
    return {k: v.architecture for k, v in sorted(_REGISTRY.items())}


def entry_for(model_type: str) -> ArchitectureEntry:
    if model_type not in _REGISTRY:
        raise ConfigError(f"unsupported model: model_type={model_type}; supported: {supported()}")
    return _REGISTRY[model_type]


def parse_config(c: Mapping[str, Any]) -> ModelConfig:
    """config.json (as a dict) -> ModelConfig.

    As model/Families.java:57-59, :95-106: ``model_type`` selects the entry; when it is missing it is
    inferred from ``architectures[0]``; a declared architecture that does not belong to the model type
    is refused with the list of what is supported.
    """
    if not isinstance(c, Mapping):
        raise ConfigError("config.json must hold a JSON object")
    archs = c.get("architectures")
    declared = str(archs[0]) if isinstance(archs, (list, tuple)) and archs else None
    model_type = c.get("model_type")
    if not isinstance(model_type, str):
        model_type = None
    if model_type is None and declared is not None:
        for k, e in _REGISTRY.items():
            if e.architecture == declared:
                model_type = k
                break
    if model_type is None or model_type not in _REGISTRY or (
            declared is not None and _REGISTRY[model_type].architecture != declared):
        raise ConfigError(f"unsupported model: model_type={model_type}, architectures={archs}; supported: {supported()}")
    e = _REGISTRY[model_type]
    return e.parse(c, model_type, declared or e.architecture)


def load_config(model_dir: str) -> ModelConfig:
    """Reads ``<model_dir>/config.json`` (model/Architecture.java:70-88); bad JSON names the file."""
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as f:
            c = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"{path}: no such file") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: {e}") from None
    return parse_config(c)
