"""Arrangements of a layer's parts around the residual stream.

"prenorm" is the reference's decoder layer
(python/lyapunov_engine/models/llama.py:125-165): h += mixer(norm1(h));
h += ffn(norm2(h)).  The adds are carried out by the norm that follows them (see
parts/base.py), so the block returns the feed-forward's output still to be
added.
"""
from __future__ import annotations

from ..config.registry import BLOCKS, FEED_FORWARDS, MIXERS, NORMS
from ..config.specs import LayerSpec
from ..kernels import ops
from .base import Block, LayerCache, StepContext


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    def __init__(self, spec: LayerSpec):
        self.names = dict(spec.names)
        self.norm1 = NORMS.build(spec.norm1)
        self.mixer = MIXERS.build(spec.mixer)
        self.norm2 = NORMS.build(spec.norm2)
        self.ffn = FEED_FORWARDS.build(spec.ffn)

    def children(self):
        n = self.names
        return {n["norm1"] + ".": self.norm1, n["mixer"] + ".": self.mixer, n["norm2"] + ".": self.norm2,
                n["ffn"] + ".": self.ffn}

    def forward(self, ctx: StepContext, h, delta, cache: LayerCache):
        x = normed(self.norm1, self.mixer, ctx, h, delta)
        a = self.mixer.forward(ctx, x, cache)
        x = normed(self.norm2, self.ffn, ctx, h, a)
        return h, self.ffn.forward(ctx, x)


def normed(norm, consumer, ctx: StepContext, h, delta):
    """h += delta; the normed rows for ``consumer``.  A norm that can and a
    consumer that takes it may pass the rows on unevaluated (ops.PendingNorm);
    a norm that does not know of pending products gets the product itself."""
    if getattr(norm, "can_defer", False):
        return norm.forward(ctx, h, delta, lazy=getattr(consumer, "takes_pending_norm", False))
    if isinstance(delta, ops.PendingLinear):
        delta = delta.run()
    return norm.forward(ctx, h, delta)
