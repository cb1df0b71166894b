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
from ..parts.base import GroupView, LayerCache, StepContext

PREFILL_TILE = 64   # new tokens of one request per workgroup of the prefill attention kernel


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


class ModelRunner:
    def __init__(self, model: DecoderModel, cache: CacheManager, pools: CachePools, dtype: torch.dtype, device):
        self.model, self.cache, self.pools = model, cache, pools
        self.dtype, self.device = dtype, torch.device(device)
        self.layout = model.cache_layout()
        self.vocab_size = model.spec.vocab_size
        self.max_position = model.spec.max_position
        self.workspace: dict = {}
        ops.require_gpu()
        # what each call of the running order gets, apart from the step's tables
        self._calls = []
        for call in model.schedule:
            g = self.layout.group_of(call.cache)
            k = v = None
            if g is not None:
                _, k, v = pools.buffer(call.cache)
            self._calls.append((g, k, v, pools.state.get(call.cache), call.writes))

    # ------------------------------------------------------------ the context
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

    def build_context_arrays(self, ids, start, count, tokens, rows) -> StepContext:
        """The same from numpy arrays: request ids (int64); the position of each
        request's first new token and the number of its new tokens (int32); all
        new tokens in the order of the requests (int32); the rows (indices into
        ``tokens``) whose logits are wanted (int32)."""
        B = len(ids)
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
        if int(ctx_len.max()) > self.max_position:
            b = int(ctx_len.argmax())
            raise StepError(f"request {int(ids[b])} would reach position {int(ctx_len[b]) - 1}, beyond the model's "
                            f"{self.max_position}")
        if int(tokens.min()) < 0 or int(tokens.max()) >= self.vocab_size:
            bad = int(np.flatnonzero((tokens < 0) | (tokens >= self.vocab_size))[0])
            b = int(np.searchsorted(q_start, bad, side="right")) - 1
            raise StepError(f"request {int(ids[b])} has a token outside the vocabulary of {self.vocab_size}")
        if rows.size and (int(rows.min()) < 0 or int(rows.max()) >= T):
            raise StepError("logits are wanted at a place the step does not bring")
        positions = np.arange(T, dtype=np.int32) + np.repeat(start - q_start[:-1], count)
        slots = np.empty(B, dtype=np.int32)

        # Attention work: tiles of PREFILL_TILE new tokens of requests that bring several, sorted by
        # (keys up to the tile's last token, request, first token): the attention kernel starts (or
        # pairs) tiles by the work they are; and the requests with one new token.
        several = np.flatnonzero(count > 1)
        dec = np.flatnonzero(count == 1).astype(np.int32)
        if several.size:
            per = (count[several] + PREFILL_TILE - 1) // PREFILL_TILE
            tile_b = np.repeat(several, per).astype(np.int32)
            first = np.cumsum(per) - per
            tile_q0 = ((np.arange(int(per.sum())) - np.repeat(first, per)) * PREFILL_TILE).astype(np.int32)
            keys = start[tile_b] + np.minimum(count[tile_b], tile_q0 + PREFILL_TILE)
            order = np.lexsort((tile_q0, tile_b, keys))
            tile_seq, tile_q0, keys = tile_b[order], tile_q0[order], keys[order]
            tile_keys = (int(keys[0]), int(keys[-1]))
        else:
            tile_seq = tile_q0 = np.zeros(0, dtype=np.int32)
            tile_keys = (0, 0)
        max_ctx_dec = int(ctx_len[dec].max()) if dec.size else 0

        sections = [tokens, positions, q_start, ctx_len, slots, rows, tile_seq, tile_q0, dec]
        group_meta = []
        for g, gc in enumerate(self.cache.groups):
            ps = gc.page_size
            width = max(1, -(-int(ctx_len.max()) // ps))
            bt = np.empty((B, width), dtype=np.int32)
            slot_map = np.empty(T, dtype=np.int32)
            try:
                self.cache.step_tables(ids, start, count, g, bt, slot_map, slots if g == 0 else None)
            except CacheError as err:
                raise StepError(str(err)) from None
            sections += [slot_map, bt.reshape(-1)]
            group_meta.append((ps, width, gc.window))

        offsets, total = [], 0
        for s in sections:
            offsets.append(total)
            total += _align4(s.size)
        host = np.zeros(max(total, 4), dtype=np.int32)
        for s, o in zip(sections, offsets):
            host[o:o + s.size] = s
        dev = torch.from_numpy(host).to(self.device)

        def view(i: int) -> torch.Tensor:
            return dev[offsets[i]:offsets[i] + sections[i].size]

        groups = []
        for g, (ps, width, window) in enumerate(group_meta):
            groups.append(GroupView(page_size=ps, block_tables=view(10 + 2 * g).view(B, width),
                                    slot_mapping=view(9 + 2 * g), max_blocks=width, window=window))
        return StepContext(
            device=self.device, dtype=self.dtype, T=T, B=B, token_ids=view(0), positions=view(1), q_start=view(2),
            ctx_len=view(3), state_slots=view(4), logit_rows=view(5), R=int(rows.size), groups=groups,
            tile_seq=view(6), tile_q0=view(7), n_tiles=int(tile_seq.size), tile_keys=tile_keys,
            dec_seqs=view(8) if dec.size else None,
            n_dec=int(dec.size), max_ctx_dec=max_ctx_dec, q_start_host=q_start.tolist(), ctx_len_host=ctx_len.tolist(),
            state_slots_host=slots.tolist(), workspace=self.workspace)

    def layer_caches(self, ctx: StepContext) -> list:
        return [LayerCache(group=ctx.groups[g] if g is not None else None, k=k, v=v, state=state, writes=writes)
                for g, k, v, state, writes in self._calls]

    # --------------------------------------------------------------- the step
    def step(self, entries: list) -> Optional[torch.Tensor]:
        """Float logits [R, vocab] in the order of the entries and of their
        ``want`` lists, or None when nothing is wanted.  The cache is written
        for every token of the step either way."""
        ctx = self.build_context(entries)
        return self.model.forward(ctx, self.layer_caches(ctx))

    def step_arrays(self, ids, start, count, tokens, rows) -> Optional[torch.Tensor]:
        """``step`` from numpy arrays (see ``build_context_arrays``)."""
        ctx = self.build_context_arrays(ids, start, count, tokens, rows)
        return self.model.forward(ctx, self.layer_caches(ctx))
