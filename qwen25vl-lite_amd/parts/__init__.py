"""The parts layers are made of.  Importing the package registers the built-in kinds."""

from . import attention, block, mlp, norm, rope, vocab  # noqa: F401  (registration)
from .base import (Block, CacheNeed, Embedding, FeedForward, GroupStep, Head, LayerSlot, Mixer, Norm, ParamSpec, Part, PartSpec,
                   PositionEncoding, ResidualStream, StateNeed, StepContext, build_part, known_parts, register_part)

__all__ = [
    "Block", "CacheNeed", "Embedding", "FeedForward", "Head", "GroupStep", "LayerSlot", "Mixer", "Norm", "ParamSpec", "Part", "PartSpec",
    "PositionEncoding", "ResidualStream", "StateNeed", "StepContext", "build_part", "known_parts", "register_part",
]
