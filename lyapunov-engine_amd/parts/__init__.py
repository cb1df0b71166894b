"""Parts of a decoder layer.  Importing the package registers the built-in ones."""
from . import attention, block, embedding, mlp, norm, rope  # noqa: F401
from .base import (Block, Embedding, FeedForward, Head, FixedStep, GroupView, LayerCache, Logits, Mixer, Norm, PagedSpec, PageTensor,
                   Part, PositionEncoding, SLOT, StateSpec, StepBatch, StepContext, StepPlan, StepPlanner, WeightSource, WeightSpec)

__all__ = ["Block", "Embedding", "Head", "FeedForward", "FixedStep", "StepBatch", "StepPlan", "StepPlanner", "GroupView", "PagedSpec", "PageTensor", "SLOT", "LayerCache", "Logits", "Mixer", "Norm", "Part",
           "PositionEncoding", "StateSpec", "StepContext", "WeightSource", "WeightSpec"]
