"""The step function: run a batch of (request, its next tokens) through the
model, from the cache, and return the logits at the wanted places.

A batch may hold any mix of prompt portions and single decoded tokens, cut
anywhere.  The reference's engine builds either an all-prompt batch, run one
prompt at a time, or an all-decode batch
(python/lyapunov_engine/engine/llm_engine.py:232-289), with
``context_lens = total_len`` and zero-padded block tables (:233-250); its model
takes ``[B, S]`` ids and positions counted from 0 (models/llama.py:196-207).
Here the batch is flat: every token carries its absolute position and its cache
slot, every request its offset, its length after the step and its block table.
The runner only reads the cache manager; taking pages (``extend``) and closing
the step (``commit``) belong to the caller, be it the scheduler or a replay.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import numpy as np
import torch

from ..cache.manager import CacheError, CacheManager, CachePools
from ..kernels import ops
from ..models.decoder import DecoderModel
from ..parts.base import FixedStep, GroupView, LayerCache, Logits, StepBatch, StepContext, StepPlan


@dataclass
class StepEntry:
    seq_id: int
    tokens: list                       # the request's next tokens
    start: int                         # absolute position of tokens[0]
    want: list = field(default_factory=list)   # indices into tokens whose logits are wanted


class StepError(ValueError):
    pass


def _align4(n: int) -> int:
    return (n + 3) & ~3


@dataclass
class StepTables:
    """One step's integers, laid out for the device: the sections of the one
    int32 buffer a step uploads (token ids, positions, request offsets and
    lengths, state slots, logit rows, per cache group a slot mapping and a
    block table, then whatever the parts' planners ask for), in host memory."""

    host: np.ndarray                   # int32: the words, sections aligned to 16 bytes
    names: list                        # section names; a planner's array is ("plan", key, name)
    sizes: list
    offsets: list
    T: int
    B: int
    R: int
    widths: list                       # block-table width per cache group
    plan_meta: dict                    # planner key -> meta
    q_start_host: list
    ctx_len_host: list
    state_slots_host: list
    fixed: Optional[FixedStep] = None

    def shape_key(self) -> tuple:
        """What a recorded step depends on beside the words themselves."""
        return (tuple(self.names), tuple(self.sizes), self.T, self.B, self.R, tuple(self.widths),
                tuple(sorted((k, tuple(sorted(m.items()))) for k, m in self.plan_meta.items())))


class _PinnedRing:
    """Pinned host buffers used in turn for the eager step's upload: a kernel
    reads the words straight from pinned memory, so the host neither stages the
    copy nor waits for it; a buffer is written again only after the kernel that
    read it last has run (an event per buffer)."""

    TURNS = 4

    def __init__(self):
        self.buffers = [None] * self.TURNS
        self.events = [None] * self.TURNS
        self.turn = 0

    def take(self, words: int) -> torch.Tensor:
        self.turn = (self.turn + 1) % self.TURNS
        if self.events[self.turn] is not None:
            self.events[self.turn].synchronize()
        buf = self.buffers[self.turn]
        if buf is None or buf.numel() < words:
            size = 1024
            while size < words:
                size *= 2
            buf = self.buffers[self.turn] = torch.zeros(size, dtype=torch.int32).pin_memory()
        return buf[:words]

    def sent(self) -> None:
        if self.events[self.turn] is None:
            self.events[self.turn] = torch.cuda.Event()
        self.events[self.turn].record()


class ModelRunner:
    def __init__(self, model: DecoderModel, cache: CacheManager, pools: CachePools, dtype: torch.dtype, device):
        self.model, self.cache, self.pools = model, cache, pools
        self.dtype, self.device = dtype, torch.device(device)
        self.layout = model.cache_layout()
        self.vocab_size = model.spec.vocab_size
        self.max_position = model.max_positions
        self.workspace: dict = {}
        self._gpu_checked = False      # the tables are host work; the device is asked for at the first launch
        # what each call of the running order gets, apart from the step's tables
        self._calls = []
        for call in model.schedule:
            g = self.layout.group_of(call.cache)
            pages = pools.buffer(call.cache)[1] if g is not None else {}
            self._calls.append((g, pages, pools.state.get(call.cache), call.writes))
        # the parts' planners, one per distinct key, in the order the parts come
        self.planners: dict = {}
        for _, part in model.named_parts():
            planner = part.step_planner()
            if planner is not None:
                self.planners.setdefault(planner.key, planner)
        self._ring = _PinnedRing()

    # ------------------------------------------------------------- the tables
    def build_context(self, entries: list) -> StepContext:
        if not entries:
            raise StepError("a step needs at least one entry")
        for e in entries:
            if len(e.tokens) == 0:
                raise StepError(f"request {e.seq_id} brings no tokens")
            if any(w < 0 or w >= len(e.tokens) for w in e.want):
                raise StepError(f"request {e.seq_id} wants logits at a place it does not bring")
        ids = np.asarray([e.seq_id for e in entries], dtype=np.int64)
        start = np.asarray([e.start for e in entries], dtype=np.int32)
        count = np.asarray([len(e.tokens) for e in entries], dtype=np.int32)
        tokens = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries])
        at, rows = 0, []
        for e in entries:
            rows += [at + w for w in e.want]
            at += len(e.tokens)
        return self.build_context_arrays(ids, start, count, tokens, np.asarray(rows, dtype=np.int32))

    def step_tables(self, ids, start, count, tokens, rows, fixed: Optional[FixedStep] = None,
                    host_for=None) -> StepTables:
        """The step's integers from numpy arrays: request ids (int64); the
        position of each request's first new token and the number of its new
        tokens (int32); all new tokens in the order of the requests (int32);
        the rows (indices into ``tokens``) whose logits are wanted (int32).

        ``fixed``: the step is (a replay of) a recorded one (see ``FixedStep``):
        the given requests are live and the rest of its rows padding; the logits
        of every request's last token are wanted (``rows`` is ignored, and
        ``count`` too in a step of one token per request), and the requests'
        pages are taken as they are (no check that a request holds exactly
        ``start`` tokens: a step started ahead of the bookkeeping runs this way).  ``host_for(words)`` supplies the host
        memory (an int32 numpy array of that length)."""
        n = len(ids)
        if fixed is None:
            B = n
            if B == 0:
                raise StepError("a step needs at least one entry")
            if len(np.unique(ids)) != B:
                raise StepError(f"a request appears twice in one step: {ids.tolist()}")
            if int(count.min()) < 1:
                raise StepError(f"request {int(ids[int(count.argmin())])} brings no tokens")
            q_start = np.zeros(B + 1, dtype=np.int32)
            np.cumsum(count, out=q_start[1:])
            T = int(q_start[-1])
            ctx_len = start + count
            if tokens.size != T:
                raise StepError(f"{tokens.size} tokens for requests that bring {T}")
            if int(tokens.min()) < 0 or int(tokens.max()) >= self.vocab_size:
                bad = int(np.flatnonzero((tokens < 0) | (tokens >= self.vocab_size))[0])
                b = int(np.searchsorted(q_start, bad, side="right")) - 1
                raise StepError(f"request {int(ids[b])} has a token outside the vocabulary of {self.vocab_size}")
            if rows.size and (int(rows.min()) < 0 or int(rows.max()) >= T):
                raise StepError("logits are wanted at a place the step does not bring")
            positions = np.arange(T, dtype=np.int32) + np.repeat(start - q_start[:-1], count)
            ctx_bound = int(ctx_len.max())
        else:
            B, T = fixed.rows, fixed.token_rows
            if n > B:
                raise StepError(f"{n} requests in a recorded step of {B} rows")
            live = np.ones(n, dtype=np.int32) if count is None or not fixed.tokens else np.asarray(count, dtype=np.int32)
            if n and int(live.min()) < 1:
                raise StepError("a request brings no tokens")
            used = int(live.sum())
            if used > T or tokens.size != used:
                raise StepError(f"{tokens.size} tokens for requests that bring {used}, in a recorded step of {T} token rows")
            count = np.zeros(B, dtype=np.int32)
            count[:n] = live
            if not fixed.tokens:
                count[n:] = 1          # a padded row of a decode step is a token row of its own
            q_start = np.zeros(B + 1, dtype=np.int32)
            np.cumsum(count, out=q_start[1:])
            first = np.zeros(B, dtype=np.int32)
            first[:n] = start
            ctx_len = np.zeros(B, dtype=np.int32)
            ctx_len[:n] = first[:n] + live
            positions = np.zeros(T, dtype=np.int32)
            positions[:used] = np.arange(used, dtype=np.int32) + np.repeat(first[:n] - q_start[:n], live)
            full = np.zeros(T, dtype=np.int32)
            full[:used] = tokens
            tokens, start = full, first
            # the logits of every request's last token (row 0 for a padded request of a prompt step)
            rows = np.maximum(q_start[1:] - 1, 0).astype(np.int32)
            ctx_bound = fixed.max_context
            if n and int(ctx_len.max()) > ctx_bound:
                raise StepError(f"a request of {int(ctx_len.max())} tokens in a step recorded for {ctx_bound}")
        if int(ctx_len.max()) > self.max_position:
            b = int(ctx_len.argmax())
            raise StepError(f"request {int(ids[b])} would reach position {int(ctx_len[b]) - 1}, beyond the "
                            f"{self.max_position} positions this engine was set up for")
        batch = StepBatch(start=start, count=count, q_start=q_start, ctx_len=ctx_len, T=T, B=B, fixed=fixed)
        plans = {key: planner.plan(batch) for key, planner in self.planners.items()}

        names = ["token_ids", "positions", "q_start", "ctx_len", "state_slots", "logit_rows"]
        sizes = [T, T, B + 1, B, B, int(rows.size)]
        widths = []
        for g, gc in enumerate(self.cache.groups):
            width = max(1, -(-ctx_bound // gc.page_size))
            widths.append(width)
            names += [("slot_mapping", g), ("block_table", g)]
            sizes += [T, B * width]
        plan_arrays = []
        for key, (arrays, _) in plans.items():
            for name, arr in arrays.items():
                if arr.dtype != np.int32 or arr.ndim != 1:
                    raise StepError(f"planner {key}: array {name!r} must be one-dimensional int32")
                names.append(("plan", key, name))
                sizes.append(int(arr.size))
                plan_arrays.append(arr)
        offsets, total = [], 0
        for size in sizes:
            offsets.append(total)
            total += _align4(size)
        total = max(total, 4)
        host = host_for(total) if host_for is not None else np.zeros(total, dtype=np.int32)
        if host.size != total:
            raise StepError(f"the step's tables take {total} words, the buffer for them has {host.size}")

        def sec(i: int) -> np.ndarray:
            return host[offsets[i]:offsets[i] + sizes[i]]

        sec(0)[:] = tokens
        sec(1)[:] = positions
        sec(2)[:] = q_start
        sec(3)[:] = ctx_len
        slots = sec(4)
        # padded rows keep their hands off every request's state: the spare slot past the last one
        slots[n:] = self.cache.num_state_slots
        sec(5)[:] = rows
        for g, gc in enumerate(self.cache.groups):
            slot_map, bt = sec(6 + 2 * g), sec(7 + 2 * g).reshape(B, widths[g])
            try:
                if fixed is None:
                    self.cache.step_tables(ids, start, count, g, bt, slot_map, slots if g == 0 else None)
                elif n:
                    ps = gc.page_size
                    self.cache.export(ids, g, bt[:n], slots[:n] if g == 0 else None)
                    used = int(q_start[n])
                    at = positions[:used]
                    slot_map[:used] = bt[np.repeat(np.arange(n), count[:n]), at // ps] * ps + at % ps
            except CacheError as err:
                raise StepError(str(err)) from None
            if fixed is not None:
                slot_map[int(q_start[n]):] = -1
        for i, arr in enumerate(plan_arrays):
            sec(len(sizes) - len(plan_arrays) + i)[:] = arr
        return StepTables(host=host, names=names, sizes=sizes, offsets=offsets, T=T, B=B, R=int(rows.size),
                          widths=widths, plan_meta={key: meta for key, (_, meta) in plans.items()},
                          q_start_host=q_start.tolist(), ctx_len_host=ctx_len.tolist(),
                          state_slots_host=slots.tolist(), fixed=fixed)

    def context(self, tables: StepTables, dev: torch.Tensor, workspace: Optional[dict] = None) -> StepContext:
        """The step as the parts see it, over ``dev``: the tables' words on the device."""
        B = tables.B

        def view(i: int) -> torch.Tensor:
            return dev[tables.offsets[i]:tables.offsets[i] + tables.sizes[i]]

        groups = []
        for g, gc in enumerate(self.cache.groups):
            groups.append(GroupView(page_size=gc.page_size, block_tables=view(7 + 2 * g).view(B, tables.widths[g]),
                                    slot_mapping=view(6 + 2 * g), max_blocks=tables.widths[g], window=gc.window))
        plans = {key: StepPlan({}, meta) for key, meta in tables.plan_meta.items()}
        for i, name in enumerate(tables.names):
            if isinstance(name, tuple) and name[0] == "plan":
                plans[name[1]].arrays[name[2]] = view(i)
        return StepContext(
            device=self.device, dtype=self.dtype, T=tables.T, B=B, token_ids=view(0), positions=view(1),
            q_start=view(2), ctx_len=view(3), state_slots=view(4), logit_rows=view(5), R=tables.R, groups=groups,
            plans=plans, q_start_host=tables.q_start_host, ctx_len_host=tables.ctx_len_host,
            state_slots_host=tables.state_slots_host, workspace=self.workspace if workspace is None else workspace,
            fixed=tables.fixed)

    def build_context_arrays(self, ids, start, count, tokens, rows) -> StepContext:
        """The eager step's context: tables written into pinned memory and read
        from there by one small kernel (see ``step_tables`` for the arguments)."""
        if not self._gpu_checked:
            ops.require_gpu()
            self._gpu_checked = True
        tables = self.step_tables(ids, start, count, tokens, rows, host_for=lambda n: self._ring.take(n).numpy())
        dev = torch.empty(tables.host.size, dtype=torch.int32, device=self.device)
        ops.table_load(self._ring.buffers[self._ring.turn], dev)
        self._ring.sent()
        return self.context(tables, dev)

    def layer_caches(self, ctx: StepContext) -> list:
        return [LayerCache(group=ctx.groups[g] if g is not None else None, pages=pages, state=state, writes=writes)
                for g, pages, state, writes in self._calls]

    # --------------------------------------------------------------- the step
    def step(self, entries: list) -> Optional[torch.Tensor]:
        """Float logits [R, vocab] in the order of the entries and of their
        ``want`` lists, or None when nothing is wanted.  The cache is written
        for every token of the step either way."""
        ctx = self.build_context(entries)
        out = self.model.forward(ctx, self.layer_caches(ctx))
        return None if out is None else out.values

    def step_arrays(self, ids, start, count, tokens, rows) -> Optional[Logits]:
        """``step`` from numpy arrays (see ``step_tables``); the result with what the head left
        for the sampler beside the values (``parts.base.Logits``)."""
        ctx = self.build_context_arrays(ids, start, count, tokens, rows)
        return self.model.forward(ctx, self.layer_caches(ctx))
