from .spec import CacheNeed, LayerSpec, ModelSpec, PartSpec, Run, WeightSpec
from .base import (CATEGORIES, Normed, PagedCacheView, Part, ResidualSink, Runtime, ScaledSum, StateCacheView, StepContext,
                   Workspace, make_part, register_part, registered_parts, unregister_part)
from . import norm, rotary, sinusoid, attention, delta, recurrent, latent, feedforward, routed, embedding, block  # register the built-in kinds

__all__ = [
    "CacheNeed", "LayerSpec", "ModelSpec", "PartSpec", "Run", "WeightSpec", "CATEGORIES",
    "Normed", "ResidualSink", "ScaledSum", "PagedCacheView", "Part", "Runtime", "StateCacheView", "StepContext", "Workspace",
    "make_part", "register_part", "registered_parts", "unregister_part",
]
