"""The parts a model is put together from, and their registries."""
from .base import BuildContext, Part, part_factory, register_part, unregister_part
from . import rope, norm, attention, ffn, block  # register the built-in parts
from .model import DecoderModel

__all__ = ["BuildContext", "Part", "part_factory", "register_part", "unregister_part", "DecoderModel"]
