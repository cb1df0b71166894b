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

from ..cache.manager import CacheManager, CachePools
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
        B = len(entries)
        seen = set()
        q_start = [0]
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.seq_id} brings no tokens")
            if e.seq_id in seen:
                raise StepError(f"request {e.seq_id} appears twice in one step")
            seen.add(e.seq_id)
            if not self.cache.has(e.seq_id):
                raise StepError(f"request {e.seq_id} is not known to the cache manager")
            if e.start != self.cache.length(e.seq_id):
                raise StepError(f"request {e.seq_id} continues at {e.start} but its cache holds "
                                f"{self.cache.length(e.seq_id)} tokens")
            if e.start + n > self.cache.capacity(e.seq_id):
                raise StepError(f"request {e.seq_id} has pages for {self.cache.capacity(e.seq_id)} tokens, "
                                f"the step needs {e.start + n}")
            if e.start + n > self.max_position:
                raise StepError(f"request {e.seq_id} would reach position {e.start + n - 1}, beyond the model's "
                                f"{self.max_position}")
            if min(e.tokens) < 0 or max(e.tokens) >= self.vocab_size:
                raise StepError(f"request {e.seq_id} has a token outside the vocabulary of {self.vocab_size}")
            if any(w < 0 or w >= n for w in e.want):
                raise StepError(f"request {e.seq_id} wants logits at a place it does not bring")
            q_start.append(q_start[-1] + n)
        T = q_start[-1]

        token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries])
        positions = np.concatenate([np.arange(e.start, e.start + len(e.tokens), dtype=np.int32) for e in entries])
        ctx_len = np.asarray([e.start + len(e.tokens) for e in entries], dtype=np.int32)
        slots = np.asarray([self.cache.state_slot(e.seq_id) for e in entries], dtype=np.int32)
        rows = np.asarray([q_start[b] + w for b, e in enumerate(entries) for w in e.want], dtype=np.int32)

        tiles, dec = [], []   # tiles: (keys up to the tile's last token, request, first token)
        for b, e in enumerate(entries):
            n = len(e.tokens)
            if n == 1:
                dec.append(b)
            else:
                for q0 in range(0, n, PREFILL_TILE):
                    tiles.append((e.start + min(n, q0 + PREFILL_TILE), b, q0))
        tiles.sort()          # the attention kernel starts (or pairs) tiles by the work they are
        tile_seq = [t[1] for t in tiles]
        tile_q0 = [t[2] for t in tiles]
        tile_keys = (tiles[0][0], tiles[-1][0]) if tiles else (0, 0)
        max_ctx_dec = max((int(ctx_len[b]) for b in dec), default=0)

        sections = [token_ids, positions, np.asarray(q_start, dtype=np.int32), ctx_len, slots, rows,
                    np.asarray(tile_seq, dtype=np.int32), np.asarray(tile_q0, dtype=np.int32),
                    np.asarray(dec, dtype=np.int32)]
        group_meta = []
        for g, gc in enumerate(self.cache.groups):
            tables = [self.cache.table(e.seq_id, g) for e in entries]
            width = max(1, max(len(t) for t in tables))
            bt = np.full((B, width), -1, dtype=np.int32)
            slot_map = np.empty(T, dtype=np.int32)
            ps = gc.page_size
            for b, (e, t) in enumerate(zip(entries, tables)):
                bt[b, :len(t)] = t
                pos = positions[q_start[b]:q_start[b + 1]]
                pages = np.asarray(t, dtype=np.int32)[pos // ps]
                if (pages < 0).any():
                    raise StepError(f"request {e.seq_id} has no page for one of its new tokens in cache group {g}")
                slot_map[q_start[b]:q_start[b + 1]] = pages * ps + pos % ps
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
            tile_seq=view(6), tile_q0=view(7), n_tiles=len(tile_seq), tile_keys=tile_keys,
            dec_seqs=view(8) if dec else None,
            n_dec=len(dec), max_ctx_dec=max_ctx_dec, q_start_host=q_start, ctx_len_host=ctx_len.tolist(),
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
