"""Parts of a decoder layer.  Importing the package registers the built-in ones."""
from . import attention, block, embedding, mlp, norm, rope  # noqa: F401
from .base import (Block, Embedding, FeedForward, Head, FixedStep, GroupView, KVCacheSpec, LayerCache, Mixer, Norm, Part,
                   PositionEncoding, StateSpec, StepBatch, StepContext, StepPlan, StepPlanner, WeightSource, WeightSpec)

__all__ = ["Block", "Embedding", "Head", "FeedForward", "FixedStep", "StepBatch", "StepPlan", "StepPlanner", "GroupView", "KVCacheSpec", "LayerCache", "Mixer", "Norm", "Part",
           "PositionEncoding", "StateSpec", "StepContext", "WeightSource", "WeightSpec"]
