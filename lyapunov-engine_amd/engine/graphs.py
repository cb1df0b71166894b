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
from ..parts.base import GroupView, StepContext
from .runner import ModelRunner, _align4


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

    def __init__(self, runner: ModelRunner, batch: int, ctx_cap: int, pool):
        self.batch, self.ctx_cap = batch, ctx_cap
        cache = runner.cache
        B = batch
        # layout of the fixed table buffer, in int32 words
        self.sizes = [B, B, B + 1, B, B, B]   # token ids, positions, q_start, ctx_len, state slots, logit rows
        self.widths = []
        for gc in cache.groups:
            width = max(1, -(-ctx_cap // gc.page_size))
            self.widths.append(width)
            self.sizes += [B, B * width]
        self.offsets, total = [], 0
        for s in self.sizes:
            self.offsets.append(total)
            total += _align4(s)
        # Several pinned copies of the table, used in turn: a step may be filled in while the copy
        # of the one before it to the device has not run yet.
        self.hosts = [torch.zeros(total, dtype=torch.int32).pin_memory() for _ in range(self.TURNS)]
        self.turn = 0
        self.dev = torch.zeros(total, dtype=torch.int32, device=runner.device)
        self.workspace: dict = {}
        self._rows = np.arange(B)
        for host in self.hosts:
            h = host.numpy()
            h[self.offsets[2]:self.offsets[2] + B + 1] = np.arange(B + 1)
            h[self.offsets[5]:self.offsets[5] + B] = np.arange(B)
        self.h = self.hosts[0].numpy()
        self.fill(runner, np.zeros(0, np.int64), np.zeros(0, np.int32), np.zeros(0, np.int32))
        self.dev.copy_(self.hosts[0])

        def view(i):
            return self.dev[self.offsets[i]:self.offsets[i] + self.sizes[i]]

        groups = [GroupView(page_size=gc.page_size, block_tables=view(7 + 2 * g).view(B, self.widths[g]),
                            slot_mapping=view(6 + 2 * g), max_blocks=self.widths[g], window=gc.window)
                  for g, gc in enumerate(cache.groups)]
        empty = self.dev[:0]
        self.ctx = StepContext(
            device=runner.device, dtype=runner.dtype, T=B, B=B, token_ids=view(0), positions=view(1), q_start=view(2),
            ctx_len=view(3), state_slots=view(4), logit_rows=view(5), R=B, groups=groups, tile_seq=empty,
            tile_q0=empty, n_tiles=0, dec_seqs=None, n_dec=B, max_ctx_dec=ctx_cap, q_start_host=list(range(B + 1)),
            ctx_len_host=[0] * B, state_slots_host=[0] * B, workspace=self.workspace)
        caches = runner.layer_caches(self.ctx)
        # One run outside the capture loads the libraries, sizes the scratch
        # buffers and lets the vendor library's algorithms for this many rows be
        # chosen by measurement, among those that need no workspace (no memset is to be
        # recorded); with every context at 0 it stores nothing in the cache.
        with ops.library_gemm_tuning(for_graph=True):
            runner.model.forward(self.ctx, caches)
            torch.cuda.synchronize()
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph, pool=pool):
                self.logits = runner.model.forward(self.ctx, caches)

    def fill(self, runner: ModelRunner, ids, starts, tokens) -> None:
        """Write the step's tables into the pinned host buffer.  ids (int64),
        starts and tokens (int32) are numpy arrays, one entry per request; rows
        past them are inert (context 0, slot -1)."""
        B, cache, h, o = self.batch, runner.cache, self.h, self.offsets
        n = len(ids)
        h[o[0]:o[0] + n] = tokens
        h[o[1]:o[1] + n] = starts
        h[o[3]:o[3] + n] = starts
        h[o[3]:o[3] + n] += 1
        for i in (0, 1, 3, 4):
            h[o[i] + n:o[i] + B] = 0
        rows = self._rows[:n]
        for g, gc in enumerate(cache.groups):
            width, ps = self.widths[g], gc.page_size
            sm = h[o[6 + 2 * g]:o[6 + 2 * g] + B]
            bt = h[o[7 + 2 * g]:o[7 + 2 * g] + B * width].reshape(B, width)
            if n:
                cache.export(ids, g, bt, h[o[4]:o[4] + n] if g == 0 else None)
                sm[:n] = bt[rows, starts // ps] * ps + starts % ps
            sm[n:] = -1

    def run(self, runner: ModelRunner, ids, starts, tokens, tokens_dev=None) -> torch.Tensor:
        """``tokens_dev``: the token ids as an int32 tensor on the device, for a
        step whose tokens the host does not know yet (``tokens`` is ignored)."""
        self.turn = (self.turn + 1) % self.TURNS
        self.h = self.hosts[self.turn].numpy()
        self.fill(runner, ids, starts, tokens)
        # one small kernel reads the pinned table (and the device's token ids) into place
        ops.table_load(self.hosts[self.turn], self.dev, None if tokens_dev is None else tokens_dev[:len(ids)],
                       self.offsets[0])
        self.graph.replay()
        return self.logits[:len(ids)]


class DecodeGraphs:
    MIN_CTX = 256

    def __init__(self, runner: ModelRunner, max_batch: int):
        self.runner = runner
        self.max_batch = _batch_bucket(max_batch)
        self.captured: dict = {}
        self.pool = None
        self.safe = all(part.graph_safe for _, part in runner.model.named_parts())

    def usable(self, entries: list) -> bool:
        return self.safe and all(len(e.tokens) == 1 and e.want == [0] for e in entries) and len(entries) <= self.max_batch

    def step(self, entries: list) -> torch.Tensor:
        """Logits [len(entries), vocab]; valid until the next graph step."""
        return self.step_arrays(np.asarray([e.seq_id for e in entries], dtype=np.int64),
                                np.asarray([e.start for e in entries], dtype=np.int32),
                                np.asarray([e.tokens[0] for e in entries], dtype=np.int32))

    def step_arrays(self, ids, starts, tokens, tokens_dev=None) -> torch.Tensor:
        """The same from numpy arrays: request ids (int64), position and id of
        each request's one new token (int32); or the ids of the tokens as a
        tensor on the device (``tokens_dev``)."""
        ctx_need = int(starts.max()) + 1
        key = (_batch_bucket(len(ids)), min(_bucket(ctx_need, self.MIN_CTX), self.runner.max_position))
        cap = self.captured.get(key)
        if cap is None:
            if self.pool is None:
                self.pool = torch.cuda.graph_pool_handle()
            cap = self.captured[key] = _Captured(self.runner, key[0], key[1], self.pool)
        return cap.run(self.runner, ids, starts, tokens, tokens_dev)
