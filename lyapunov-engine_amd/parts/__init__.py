"""Parts of a decoder layer.  Importing the package registers the built-in ones."""
from . import attention, block, mlp, norm, rope  # noqa: F401
from .base import (Block, FeedForward, GroupView, KVCacheSpec, LayerCache, Mixer, Norm, Part, PositionEncoding,
                   StateSpec, StepContext, WeightSource, WeightSpec)

__all__ = ["Block", "FeedForward", "GroupView", "KVCacheSpec", "LayerCache", "Mixer", "Norm", "Part",
           "PositionEncoding", "StateSpec", "StepContext", "WeightSource", "WeightSpec"]
