from .spec import CacheNeed, LayerSpec, ModelSpec, PartSpec, Run, WeightSpec
from .base import (CATEGORIES, Normed, PagedCacheView, Part, ResidualSink, Runtime, StateCacheView, StepContext,
                   Workspace, make_part, register_part, registered_parts, unregister_part)
from . import norm, rotary, attention, feedforward, embedding, block  # register the built-in kinds

__all__ = [
    "CacheNeed", "LayerSpec", "ModelSpec", "PartSpec", "Run", "WeightSpec", "CATEGORIES",
    "Normed", "ResidualSink", "PagedCacheView", "Part", "Runtime", "StateCacheView", "StepContext", "Workspace",
    "make_part", "register_part", "registered_parts", "unregister_part",
]
