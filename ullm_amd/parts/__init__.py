"""Parts a layer is put together from.  Importing the package registers the built-in parts."""
from .base import (Block, CacheNeed, CacheRows, FeedForward, GroupView, KVNeed, LayerCache, Mixer, Norm, Part, PartEnv,
                   PendingNorm, PositionEncoding, StateNeed, StepContext, StepPlan, StepShape, WeightDecl, build_part,
                   register_part, registered_parts, walk, cache_needs_of)
from . import norm, position, attention, feedforward, block  # noqa: F401  (registration)

__all__ = ["Block", "CacheNeed", "CacheRows", "StepPlan", "StepShape", "FeedForward", "GroupView", "KVNeed", "LayerCache", "Mixer", "Norm", "Part",
           "PartEnv", "PendingNorm", "PositionEncoding", "StateNeed", "StepContext", "WeightDecl", "build_part",
           "register_part", "registered_parts", "walk", "cache_needs_of"]
