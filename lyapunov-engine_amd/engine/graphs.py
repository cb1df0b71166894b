"""Decode steps replayed from captured HIP graphs.

A step in which every request brings exactly one token launches some hundred
small kernels; launched one by one from Python, the launches cost more than the
kernels.  Such steps are captured once per (batch bucket, context bucket) and
replayed: a small kernel reads the step's tables from pinned host memory into
fixed device buffers (the token ids from the sampler's device buffer when the
host does not know them yet), the graph runs, the logits are read from a fixed
tensor.

The reference buckets by batch size {1, 2, 4, ... 64}, takes the smallest bucket
that fits, pads with zeros and slices the result
(python/lyapunov_engine/engine/cuda_graph_runner.py:15-16, 59-80; the C++ runner,
csrc/engine/cuda_graph.cpp:15-68, warms up once and then captures).  Its graph
holds a model call without a cache (cuda_graph_runner.py:43-49).  Here the graph
holds the real step over the paged cache; padded rows have a context of 0 (the
attention kernels skip them) and a cache slot of -1 (nothing is stored).  The
context bucket bounds the width of the block tables and the number of attention
partitions a launch provides for.

Nothing that clears memory with a memset is recorded: the kernels write every
value they later read.
"""
from __future__ import annotations

import numpy as np
import torch

from ..kernels import ops
from ..parts.base import FixedStep, Logits
from .runner import ModelRunner, StepError


class RecordingFailed(RuntimeError):
    """A step could not be recorded for lack of a resource (device memory, the
    graph itself): the one failure of a recorded step that the engine answers
    by stepping eagerly.  Errors in the tables or from a kernel's checks are
    not of this kind and are raised as they are."""


def _bucket(n: int, smallest: int) -> int:
    b = smallest
    while b < n:
        b *= 2
    return b


def _batch_bucket(n: int) -> int:
    """Batch sizes a graph is captured for: 1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48,
    64, ...  A step pays for its padded rows nearly as for real ones (33
    requests in a graph of 64 took 19 % longer than 32 in one of 32), so the
    steps between powers of two (the reference's buckets) get graphs too."""
    b = _bucket(n, 1)
    return b * 3 // 4 if b >= 4 and n <= b * 3 // 4 else b


class _Captured:
    TURNS = 3

    def __init__(self, runner: ModelRunner, fixed: FixedStep, pool):
        self.fixed = fixed
        none64, none32 = np.zeros(0, np.int64), np.zeros(0, np.int32)
        # The step function lays the tables out, as for any step; with no live request every row is
        # padding (context 0, slot -1), so the runs below store nothing in the cache.
        first = runner.step_tables(none64, none32, None, none32, None, fixed=self.fixed)
        self.shape = first.shape_key()
        self.token_words = first.offsets[0]
        words = first.host.size
        # Several pinned copies of the table, used in turn: a step may be filled in while the copy
        # of the one before it to the device has not run yet.
        self.hosts = [torch.zeros(words, dtype=torch.int32).pin_memory() for _ in range(self.TURNS)]
        self.turn = 0
        self.hosts[0].numpy()[:] = first.host
        self.dev = torch.zeros(words, dtype=torch.int32, device=runner.device)
        self.dev.copy_(self.hosts[0])
        self.workspace: dict = {}
        self.ctx = runner.context(first, self.dev, workspace=self.workspace)
        caches = runner.layer_caches(self.ctx)
        # One run outside the capture loads the libraries, sizes the scratch
        # buffers and lets the vendor library's algorithms for this many rows be
        # chosen by measurement, among those that need no workspace (no memset is to be
        # recorded).
        with ops.library_gemm_tuning(for_graph=True):
            try:
                runner.model.forward(self.ctx, caches)
                torch.cuda.synchronize()
                self.graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(self.graph, pool=pool):
                    self.logits = runner.model.forward(self.ctx, caches)
            except ops.KernelError:
                raise                      # a kernel's own check: a defect, not a shortage
            except (torch.cuda.OutOfMemoryError, RuntimeError) as err:   # what torch raises when memory or the capture fails
                raise RecordingFailed(f"{fixed}: {type(err).__name__}: {err}") from err

    def run(self, runner: ModelRunner, ids, starts, tokens, tokens_dev=None, counts=None) -> Logits:
        """``tokens_dev``: the token ids as an int32 tensor on the device, for a
        step whose tokens the host does not know yet (``tokens`` is ignored).
        ``counts``: new tokens per request, for a recorded step with prompt tokens."""
        self.turn = (self.turn + 1) % self.TURNS
        host = self.hosts[self.turn]
        tables = runner.step_tables(ids, starts, counts, tokens, None, fixed=self.fixed, host_for=lambda n: host.numpy())
        if tables.shape_key() != self.shape:
            raise StepError("a planner's arrays or launch shapes changed between two steps of one recorded shape: "
                            "in a fixed step they may depend on the step's bounds alone")
        # one small kernel reads the pinned table (and the device's token ids) into place
        ops.table_load(host, self.dev, None if tokens_dev is None else tokens_dev[:len(ids)], self.token_words)
        self.graph.replay()
        return self.logits.first(len(ids))


class StepGraphs:
    """Recorded steps of a model, by shape: decode steps (every request one
    token) per (batch bucket, context bucket), and short prompt steps (one
    request, up to ``PROMPT_TOKENS[-1]`` tokens, nothing else in the step) per
    (token bucket, context bucket): a prompt of a few tokens is as much bound
    by its launches as a decode step is."""

    MIN_CTX = 256
    PROMPT_TOKENS = (16, 32, 64, 128)   # token rows a recorded prompt step may have

    def __init__(self, runner: ModelRunner, max_batch: int):
        self.runner = runner
        self.max_batch = _batch_bucket(max_batch)
        self.captured: dict = {}
        self.pool = None
        self.safe = all(part.graph_safe for _, part in runner.model.named_parts())

    def usable(self, entries: list) -> bool:
        return self.safe and all(len(e.tokens) == 1 and e.want == [0] for e in entries) and len(entries) <= self.max_batch

    def _captured(self, fixed: FixedStep) -> _Captured:
        key = (fixed.rows, fixed.max_context) if not fixed.tokens else (fixed.rows, fixed.max_context, fixed.tokens)
        cap = self.captured.get(key)
        if cap is None:
            if self.pool is None:
                self.pool = torch.cuda.graph_pool_handle()
            cap = self.captured[key] = _Captured(self.runner, fixed, self.pool)
        return cap

    def _context_bucket(self, ctx_need: int) -> int:
        return min(_bucket(ctx_need, self.MIN_CTX), self.runner.max_position)

    def step(self, entries: list) -> torch.Tensor:
        """Logits [len(entries), vocab]; valid until the next graph step."""
        return self.step_arrays(np.asarray([e.seq_id for e in entries], dtype=np.int64),
                                np.asarray([e.start for e in entries], dtype=np.int32),
                                np.asarray([e.tokens[0] for e in entries], dtype=np.int32)).values

    def step_arrays(self, ids, starts, tokens, tokens_dev=None) -> Logits:
        """The same from numpy arrays: request ids (int64), position and id of
        each request's one new token (int32); or the ids of the tokens as a
        tensor on the device (``tokens_dev``).  Returns the rows' ``Logits``."""
        fixed = FixedStep(rows=_batch_bucket(len(ids)), max_context=self._context_bucket(int(starts.max()) + 1))
        return self._captured(fixed).run(self.runner, ids, starts, tokens, tokens_dev)

    def prompt_usable(self, count) -> bool:
        """Whether a step of these new-token counts (one per request) is one that is recorded as a
        prompt step: one request, more than one token, no more than the largest bucket."""
        return self.safe and len(count) == 1 and 1 < int(count[0]) <= self.PROMPT_TOKENS[-1]

    def prompt_step_arrays(self, ids, starts, counts, tokens) -> Logits:
        """A short prompt (or its last portion) alone in a step: logits [1, vocab] of its last token."""
        rows = next(t for t in self.PROMPT_TOKENS if t >= int(counts.sum()))
        fixed = FixedStep(rows=len(ids), max_context=self._context_bucket(int((starts + counts).max())), tokens=rows)
        return self._captured(fixed).run(self.runner, ids, starts, tokens, counts=counts)


DecodeGraphs = StepGraphs
