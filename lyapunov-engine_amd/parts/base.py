"""Interfaces of the parts a decoder layer is made of, and of what a step hands
to them.

A part is built from sizes and constants alone (never from a model name), says
which tensors it wants (``weight_specs``), what it needs from the cache
(``cache_spec`` / ``state_spec``, mixers only), and computes in ``forward``.
The model builder looks parts up in the registries of ``config.registry``; a
part defined anywhere (a test, another package) that follows these interfaces
and registers itself can be used by a ModelSpec without touching this package.

Conventions every part may rely on:
  * the hidden state ``h`` is the float residual stream ``[T, hidden]``;
    a part's output ``y`` has the step's activation dtype (``ctx.dtype``) and is
    added to ``h`` by the *next* norm (``Norm.forward(ctx, h, delta=y)``), in
    32-bit; ``y`` may also be float partial sums ``[S, T, hidden]`` (what
    ``ops.linear(..., may_split=True)`` returns), which that norm adds up;
  * ``T`` is the number of tokens of the step, all requests' tokens flattened;
    request ``b`` owns rows ``q_start[b] .. q_start[b+1]``, in position order;
  * a part's result for a token may depend on earlier tokens of the same request
    (through the cache it is handed) and on nothing else in the batch.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional

import numpy as np
import torch


# --------------------------------------------------------------------- weights
@dataclass(frozen=True)
class WeightSource:
    name: str              # tensor name in the file, relative to the part's prefix
    shape: tuple


@dataclass(frozen=True)
class WeightSpec:
    """One tensor of a part: attribute ``attr`` receives the sources
    concatenated along dimension 0 (one source: the tensor itself)."""

    attr: str
    sources: tuple         # of WeightSource
    init: str = "normal"   # random-weights mode: "normal" (0, std) or "ones" (1 + noise)
    interleave: int = 0    # n > 0: rows alternate between the sources in runs of n (n of the first, n of the second, ...)

    @property
    def shape(self) -> tuple:
        first = self.sources[0].shape
        return (sum(s.shape[0] for s in self.sources),) + tuple(first[1:])


class Part:
    """Anything that may own weights and sub-parts."""

    # False for a part whose forward reads the host copies of the step's tables
    # (``ctx.q_start_host`` and the like) or lets the device's values decide
    # what is launched: such a forward cannot be recorded once and replayed with
    # other tables, so its model steps eagerly.  A part that needs lists of its
    # own on the device gets them through ``step_planner`` and stays graph-safe.
    graph_safe = True

    def weight_specs(self) -> list:
        return []

    def children(self) -> dict:
        """Sub-parts by the piece of tensor-name prefix that leads to them
        (for example ``{"q_norm.": self.q_norm}``)."""
        return {}

    def materialize(self, device: torch.device, dtype: torch.dtype) -> None:
        """Build device tables that are computed rather than loaded."""
        for c in self.children().values():
            c.materialize(device, dtype)

    def step_planner(self) -> Optional["StepPlanner"]:
        """What this part wants worked out once per step, on the host, from the
        step's requests (see ``StepPlanner``); None: nothing."""
        return None


# ----------------------------------------------------------------------- cache
SLOT = -1   # in a PageTensor's shape: the dimension that runs over the token slots of a page


@dataclass(frozen=True)
class PageTensor:
    """One of the tensors a mixer keeps per token in pages.  ``shape`` is the
    shape of one page with ``SLOT`` where the page's token slots run (its
    extent is the group's page size): ``(heads, SLOT, head_dim)`` keeps a
    token's values side by side, ``(heads, head_dim, SLOT)`` keeps the slots of
    one dimension side by side.  ``dtype`` None: the engine's activation type."""

    name: str
    shape: tuple
    dtype: Optional[torch.dtype] = None

    def page_shape(self, page_size: int) -> tuple:
        if self.shape.count(SLOT) != 1:
            raise ValueError(f"page tensor {self.name!r}: exactly one dimension is the token slot, got {self.shape}")
        return tuple(page_size if d == SLOT else int(d) for d in self.shape)


@dataclass(frozen=True)
class PagedSpec:
    """What a mixer keeps per token, in pages: the layout is the mixer's, the
    pages, block tables and their reuse are the cache manager's.  Calls whose
    specs are equal share a group: one pool of pages, one block table per
    request."""

    tensors: tuple         # of PageTensor
    window: int = 0        # 0: every token is kept; W: a token needs the last W tokens' entries, its own included

    @classmethod
    def keys_and_values(cls, num_kv_heads: int, head_dim: int, window: int = 0) -> "PagedSpec":
        """The layout the attention kernels of this package read: keys
        [heads][slot][head_dim], values [heads][head_dim][slot]."""
        return cls((PageTensor("k", (num_kv_heads, SLOT, head_dim)), PageTensor("v", (num_kv_heads, head_dim, SLOT))),
                   int(window))


@dataclass(frozen=True)
class StateSpec:
    """State of fixed size per live request (a slot of ``shape``), for mixers
    that carry a summary instead of keys."""

    shape: tuple
    dtype: torch.dtype = torch.float32


@dataclass
class GroupView:
    """A cache group as a step sees it."""

    page_size: int
    block_tables: torch.Tensor        # int32 [B, max_blocks]; -1 where a page was given back
    slot_mapping: torch.Tensor        # int32 [T]: page * page_size + offset of each new token
    max_blocks: int
    window: int = 0


@dataclass
class LayerCache:
    """What one call of a layer gets from the cache."""

    group: Optional[GroupView] = None
    pages: dict = field(default_factory=dict)   # PageTensor.name -> [pages, *PageTensor.page_shape(page size)]
    state: Optional[torch.Tensor] = None  # [slots, *StateSpec.shape]
    writes: bool = True                   # false: read what another call stored

    @property
    def k(self) -> Optional[torch.Tensor]:
        """The pool named "k" (``PagedSpec.keys_and_values``: [pages, kv heads, page_size, head_dim])."""
        return self.pages.get("k")

    @property
    def v(self) -> Optional[torch.Tensor]:
        """The pool named "v" ([pages, kv heads, head_dim, page_size])."""
        return self.pages.get("v")


@dataclass
class FixedStep:
    """A step whose shapes are frozen so that it can be recorded once and
    replayed.  ``tokens == 0``: ``rows`` requests of one new token each (rows
    past the live ones are padding: context 0, cache slot -1, the spare state
    slot).  ``tokens > 0``: up to ``rows`` requests that bring up to ``tokens``
    new tokens between them, a request's tokens side by side as in any step;
    the token rows past the live ones are padding (position 0, cache slot -1,
    owned by no request), and so are requests past the live ones (no tokens,
    context 0).  Contexts are at most ``max_context`` tokens either way."""

    rows: int
    max_context: int
    tokens: int = 0

    @property
    def token_rows(self) -> int:
        return self.tokens or self.rows


@dataclass
class StepBatch:
    """The requests of a step as the host sees them (numpy), for planners."""

    start: np.ndarray                     # int32 [B]: position of each request's first new token
    count: np.ndarray                     # int32 [B]: how many new tokens it brings
    q_start: np.ndarray                   # int32 [B + 1]: offsets into the flat batch
    ctx_len: np.ndarray                   # int32 [B]: length after the step (0: a padded row of a fixed step)
    T: int
    B: int
    fixed: Optional[FixedStep] = None


class StepPlanner:
    """Host work a part wants done once per step: from the step's requests to
    the lists its kernels walk (tiles, queues, segment tables).  The step
    function calls ``plan`` once per step and distinct ``key`` (parts whose
    planners have equal keys share one plan), sends the arrays to the device in
    the step's one upload, and hands the part a ``StepPlan`` under
    ``ctx.plans[key]``.

    For a fixed step (``batch.fixed``) the sizes of the arrays and every value
    of ``meta`` may depend on ``batch.fixed`` alone, never on the live
    requests: the kernels' launch shapes are recorded once; the arrays'
    contents are written afresh before every replay."""

    key: tuple = ()

    def plan(self, batch: StepBatch) -> tuple:
        """-> (arrays, meta): int32 numpy arrays by name, and host values
        (launch shapes, counts) by name."""
        raise NotImplementedError


@dataclass
class StepPlan:
    arrays: dict                          # name -> int32 tensor on the device
    meta: dict                            # name -> host value


@dataclass
class StepContext:
    """Everything about the batch of one step, on the device and on the host."""

    device: torch.device
    dtype: torch.dtype                    # activation dtype of the step
    T: int
    B: int
    token_ids: torch.Tensor               # int32 [T]
    positions: torch.Tensor               # int32 [T] absolute positions
    q_start: torch.Tensor                 # int32 [B + 1]
    ctx_len: torch.Tensor                 # int32 [B] length of each request after the step
    state_slots: torch.Tensor             # int32 [B]
    logit_rows: torch.Tensor              # int32 [R] rows of the flat batch whose logits are wanted
    R: int
    groups: list                          # of GroupView
    plans: dict = field(default_factory=dict)       # StepPlanner.key -> StepPlan
    # host copies for parts written in Python (a part that reads them is not graph_safe)
    q_start_host: list = field(default_factory=list)
    ctx_len_host: list = field(default_factory=list)
    state_slots_host: list = field(default_factory=list)
    workspace: dict = field(default_factory=dict)   # scratch tensors shared by the layers of a step
    fixed: Optional[FixedStep] = None     # set while a fixed step is recorded or replayed

    def scratch(self, key: str, numel: int, dtype: torch.dtype = torch.float32) -> torch.Tensor:
        t = self.workspace.get(key)
        if t is None or t.numel() < numel or t.dtype != dtype:
            t = torch.empty(max(numel, 1), dtype=dtype, device=self.device)
            self.workspace[key] = t
        return t


# ------------------------------------------------------------------ part kinds
class Norm(Part):
    # True: ``forward`` also takes ``lazy`` and a delta that is a product still
    # to be run (kernels.ops.PendingLinear), and with ``lazy`` may return the
    # rows undone, as a kernels.ops.PendingNorm.  False: the block resolves such
    # a delta first; the delta is then a tensor [T, H] in the activations' type
    # or float partial sums [S, T, H] (kernels.ops.as_delta makes one tensor of
    # either).
    can_defer = False

    def forward(self, ctx: StepContext, h: torch.Tensor, delta: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Add ``delta`` to ``h`` (in place, 32-bit), norm, return activations.
        With ``rows`` only those rows are normed and ``h`` is left alone."""
        raise NotImplementedError


class Embedding(Part):
    """From token ids to the residual stream's first value.  ``weight`` is the
    matrix [vocab, hidden] that a tied output head uses as its own."""

    weight: Optional[torch.Tensor] = None

    def forward(self, ctx: StepContext, token_ids: torch.Tensor) -> torch.Tensor:
        """float [T, hidden] for int32 ``token_ids`` [T]."""
        raise NotImplementedError


@dataclass
class Logits:
    """What a step returns for the rows whose logits were wanted: the float
    logits [R, vocab] and, when the head's kernel produced them on its way,
    ``row_maxima``: int32 [R, pieces, 2], for every row the largest logit
    (its bits) and the first place it stands at within each of ``pieces``
    stretches of the vocabulary.  The sampler uses them instead of a pass over
    the row; a head that changes the logits after its product (a bias, a cap)
    returns none, or ones that hold for the changed values."""

    values: torch.Tensor
    row_maxima: Optional[torch.Tensor] = None

    def first(self, n: int) -> "Logits":
        """The first ``n`` rows (views)."""
        return Logits(self.values[:n], None if self.row_maxima is None else self.row_maxima[:n])


class Head(Part):
    """From the normed rows whose logits are wanted to float logits [R, vocab]:
    ``forward`` returns a ``Logits``, or just the tensor of values."""

    def tie(self, embedding: Embedding) -> None:
        """The model ties its head to the embedding: use ``embedding.weight``
        (available from ``materialize`` on) and own no matrix.  A head that
        cannot raises."""
        raise NotImplementedError(f"{type(self).__name__} cannot share the embedding's matrix")

    def forward(self, ctx: StepContext, x: torch.Tensor) -> "Logits | torch.Tensor":
        raise NotImplementedError


class PositionEncoding(Part):
    """Turns positions into whatever the mixer applies.  The rotary kind exposes
    ``table`` (float [max_position, rotary_dim]: cosines then sines)."""

    table: Optional[torch.Tensor] = None
    rotary_dim: int = 0

    def limit_positions(self, n: int) -> None:
        """Called before ``materialize`` when the engine will never reach
        position ``n``: tables need no more rows than that."""


class Mixer(Part):
    """Mixes information between the tokens of a request.  What ``forward``
    returns is only ever added to the residual stream: a tensor [T, H], float
    partial sums [S, T, H] or a kernels.ops.PendingLinear."""

    # True: ``x`` may arrive as a kernels.ops.PendingNorm (normed rows not yet
    # computed), which the part's first product folds in.
    takes_pending_norm = False

    def cache_spec(self) -> Optional[PagedSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def forward(self, ctx: StepContext, x: torch.Tensor, cache: LayerCache) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    takes_pending_norm = False   # as for Mixer

    def forward(self, ctx: StepContext, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """Arrangement of a mixer, a feed-forward and their norms around the
    residual stream."""

    mixer: Mixer

    def forward(self, ctx: StepContext, h: torch.Tensor, delta: Optional[torch.Tensor],
                cache: LayerCache) -> tuple:
        """-> (h, delta): the residual stream and the output not yet added to it."""
        raise NotImplementedError


__all__ = [
    "WeightSource", "WeightSpec", "Part", "PagedSpec", "PageTensor", "SLOT", "StateSpec", "GroupView", "LayerCache", "StepContext",
    "StepBatch", "StepPlan", "StepPlanner", "FixedStep",
    "Norm", "PositionEncoding", "Mixer", "FeedForward", "Block", "Logits", "Any",
]
