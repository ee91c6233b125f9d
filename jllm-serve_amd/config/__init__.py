"""Typed configuration: schema records, the architecture registry, the Qwen3 parser."""
from .schema import (ConfigError, GatedMlpNames, GatedMlpSpec, GqaNames, GqaSpec, LayerSpec, ModelConfig, ModelNames,
                     NormSpec, RopeScaling, RopeSpec, ScheduleEntry, default_schedule)
from .registry import (entry_for, load_config, parse_config, register_architecture, supported,
                       unregister_architecture)
from . import qwen3 as _qwen3  # registers "qwen3"

__all__ = ["ConfigError", "GatedMlpNames", "GatedMlpSpec", "GqaNames", "GqaSpec", "ModelNames", "LayerSpec", "ModelConfig", "NormSpec", "RopeScaling", "RopeSpec",
           "ScheduleEntry", "default_schedule", "entry_for", "load_config", "parse_config", "register_architecture",
           "supported", "unregister_architecture"]
