"""A decoder put together from a ModelSpec: embedding, the layers in their
running order, final norm, output head, each looked up by its kind.

The order of work is the reference's LlamaForCausalLM.forward
(python/lyapunov_engine/models/llama.py:196-225): embed, layers, final norm,
lm_head.  Differences: the batch is flat (tokens of several requests, each with
its position), the final norm and the head run only on the rows whose logits are
wanted (the reference computes all positions and the engine keeps the last,
engine/llm_engine.py:272, 289), logits are float, and a tied head is the
embedding matrix itself, not a copy (models/weight_loader.py:106-109 copies).
"""
from __future__ import annotations

import fnmatch
from dataclasses import dataclass
from typing import Iterator, Optional

import torch

from ..config.registry import BLOCKS, EMBEDDINGS, HEADS, NORMS
from ..config.specs import LayerCall, ModelSpec
from ..kernels import ops
from ..parts.base import (LayerCache, Logits, PagedSpec, Part, PositionEncoding, StateSpec, StepContext, WeightSource,
                          WeightSpec)


@dataclass(frozen=True)
class CacheGroupLayout:
    spec: PagedSpec
    buffers: tuple          # cache ids (LayerCall.cache) whose keys and values live in this group


@dataclass(frozen=True)
class CacheLayout:
    groups: tuple           # of CacheGroupLayout
    states: dict            # cache id -> StateSpec

    def group_of(self, cache_id: int) -> Optional[int]:
        for g, layout in enumerate(self.groups):
            if cache_id in layout.buffers:
                return g
        return None


class DecoderModel(Part):
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = EMBEDDINGS.build(spec.embedding, vocab_size=spec.vocab_size, hidden_size=spec.hidden_size)
        self.layers = [BLOCKS.get(ls.block)(ls) for ls in spec.layers]
        self.final_norm = NORMS.build(spec.final_norm)
        self.head = HEADS.build(spec.head, vocab_size=spec.vocab_size, hidden_size=spec.hidden_size)
        if spec.tie_word_embeddings:
            self.head.tie(self.embedding)
        self.schedule: tuple = tuple(spec.schedule)
        for call in self.schedule:
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"the running order names layer {call.layer}; there are {len(self.layers)}")
        self.device: Optional[torch.device] = None
        self.dtype: Optional[torch.dtype] = None
        self.max_positions = spec.max_position      # positions a step may reach; ``materialize`` may lower it
        self._layout = self._plan_cache()

    @property
    def embed(self) -> Optional[torch.Tensor]:
        """The embedding's matrix."""
        return self.embedding.weight

    @property
    def lm_head(self) -> Optional[torch.Tensor]:
        """The output head's matrix (the embedding's when they are tied)."""
        return getattr(self.head, "weight", None)

    # -------------------------------------------------------------- structure
    def named_parts(self) -> Iterator[tuple]:
        """(tensor-name prefix, part) for every part that may own weights."""
        def walk(prefix: str, part: Part):
            yield prefix, part
            for piece, child in part.children().items():
                yield from walk(prefix + piece, child)

        yield from walk(self.spec.embed_prefix, self.embedding)
        for i, layer in enumerate(self.layers):
            yield from walk(self.spec.layer_prefix.format(i=i), layer)
        yield from walk(self.spec.final_norm_prefix, self.final_norm)
        yield from walk(self.spec.head_prefix, self.head)

    def weight_table(self) -> list:
        """(owner, WeightSpec with full tensor names) for the whole model."""
        out = []
        for prefix, part in self.named_parts():
            for ws in part.weight_specs():
                full = tuple(WeightSource(prefix + s.name, tuple(s.shape)) for s in ws.sources)
                out.append((part, WeightSpec(ws.attr, full, ws.init, ws.interleave)))
        return out

    def expected_tensors(self) -> dict:
        """Tensor name in the model file -> (shape, init kind)."""
        out = {}
        for _, ws in self.weight_table():
            for s in ws.sources:
                if s.name in out:
                    raise ValueError(f"two parts claim the tensor {s.name!r}")
                out[s.name] = (tuple(s.shape), ws.init)
        return out

    def ignorable(self, name: str) -> bool:
        """Whether a file may hold this tensor without the model using it: a
        tied model's separate head, and what the architecture declares
        (``ModelSpec.ignorable_tensors``: shell-style patterns, for buffers that
        exporters write and that are computed here, not loaded)."""
        if self.spec.tie_word_embeddings and name.startswith(self.spec.head_prefix):
            return True
        return any(fnmatch.fnmatchcase(name, pat) for pat in self.spec.ignorable_tensors)

    def _plan_cache(self) -> CacheLayout:
        by_cache: dict = {}
        states: dict = {}
        for call in self.schedule:
            mixer = self.layers[call.layer].mixer
            kv, st = mixer.cache_spec(), mixer.state_spec()
            if kv is not None:
                if call.cache in by_cache and by_cache[call.cache] != kv:
                    raise ValueError(f"cache buffer {call.cache} is used with two shapes: {by_cache[call.cache]} and {kv}")
                by_cache.setdefault(call.cache, kv)
            if st is not None:
                if call.cache in states and states[call.cache] != st:
                    raise ValueError(f"state buffer {call.cache} is used with two shapes")
                states.setdefault(call.cache, st)
        written = {c.cache for c in self.schedule if c.writes}
        for call in self.schedule:
            if not call.writes and call.cache not in written:
                raise ValueError(f"layer call reads cache buffer {call.cache}, which no call writes")
        order: list = []
        for call in self.schedule:  # groups in order of first use
            kv = by_cache.get(call.cache)
            if kv is not None and kv not in order:
                order.append(kv)
        groups = tuple(CacheGroupLayout(kv, tuple(sorted(c for c, s in by_cache.items() if s == kv))) for kv in order)
        return CacheLayout(groups, states)

    def cache_layout(self) -> CacheLayout:
        return self._layout

    # ---------------------------------------------------------------- weights
    def materialize(self, device, dtype, max_positions: Optional[int] = None):
        """Build what is computed rather than loaded.  ``max_positions``: the
        engine will never hold a request longer than this (its model length, its
        pool), so position tables need no more rows."""
        self.device, self.dtype = torch.device(device), dtype
        if max_positions is not None:
            self.max_positions = max(1, min(self.spec.max_position, int(max_positions)))
            for _, part in self.named_parts():
                if isinstance(part, PositionEncoding):
                    part.limit_positions(self.max_positions)
        self.embedding.materialize(self.device, dtype)
        for layer in self.layers:
            layer.materialize(self.device, dtype)
        self.final_norm.materialize(self.device, dtype)
        self.head.materialize(self.device, dtype)

    # ---------------------------------------------------------------- compute
    def forward(self, ctx: StepContext, caches: list) -> Optional[Logits]:
        """Run the step's tokens through every call of the running order;
        returns the float logits [R, vocab] for ``ctx.logit_rows`` as a
        ``Logits`` (None if R == 0).
        ``caches[i]`` is the LayerCache of ``schedule[i]``."""
        h = self.embedding.forward(ctx, ctx.token_ids)
        delta = None
        for call, cache in zip(self.schedule, caches):
            h, delta = self.layers[call.layer].forward(ctx, h, delta, cache)
        if ctx.R == 0:
            return None
        if isinstance(delta, ops.PendingLinear) and not getattr(self.final_norm, "can_defer", False):
            delta = delta.run()
        x = self.final_norm.forward(ctx, h, delta, rows=ctx.logit_rows)
        out = self.head.forward(ctx, x)
        return out if isinstance(out, Logits) else Logits(out)


def build_model(spec: ModelSpec) -> DecoderModel:
    return DecoderModel(spec)


__all__ = ["DecoderModel", "CacheLayout", "CacheGroupLayout", "build_model", "LayerCall", "StateSpec"]
