"""Grouped-query attention over the paged cache.

The reference's LlamaAttention (python/lyapunov_engine/models/llama.py:34-106):
q/k/v/o projections without bias, rotation of q and k, query head h reading
key/value head h // g, scale 1/sqrt(head_dim), causal.  The reference keeps
q_proj, k_proj and v_proj apart and never stores k and v (llama.py:82-104 drops
them after a prompt); here the three are one matrix, and every token's key and
value go into the request's pages before attention reads from the pages, so a
whole prompt, a portion of one and a decoded token take the same path.

Options beyond the reference: a window (a token sees the last W keys), no
rotation, a rotation of part of the head, and ``own_kv=False`` for a layer that
reads the keys and values another layer stored.
"""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch

from ..config.registry import MIXERS, POSITION_ENCODINGS
from ..config.specs import PartSpec
from ..kernels import ops
from .base import LayerCache, PagedSpec, Mixer, StepBatch, StepContext, StepPlanner, WeightSource, WeightSpec

PREFILL_TILE = 64   # new tokens of one request per workgroup of the prefill attention kernel


class AttentionWork(StepPlanner):
    """The attention kernels' work lists for a step.  Requests that bring
    several tokens are cut into tiles of PREFILL_TILE tokens, sorted by (keys up
    to the tile's last token, request, first token): the prefill kernel starts
    (or pairs) tiles by the work they are.  Requests that bring one token go to
    the split kernel.

    arrays: ``tile_seq``, ``tile_q0`` (request and first token of every tile),
    ``dec`` (the one-token requests; absent when there are none, and in a fixed
    step, where every row is one).  meta: ``n_tiles``, ``tile_keys`` (keys seen
    by the first and by the last tile), ``n_dec``, ``max_ctx_dec`` (the longest
    context among the one-token requests; in a fixed step the step's bound)."""

    key = ("paged_attention_work", PREFILL_TILE)

    def plan(self, batch: StepBatch) -> tuple:
        none = np.zeros(0, dtype=np.int32)
        fixed = batch.fixed
        if fixed is not None and not fixed.tokens:
            return ({"tile_seq": none, "tile_q0": none},
                    dict(n_tiles=0, tile_keys=(0, 0), n_dec=fixed.rows, max_ctx_dec=fixed.max_context))
        if fixed is not None:
            # A recorded step with prompt tokens: every request goes in tiles (one with a single
            # token too), in as many list entries as the step can ever need; entries past the live
            # tiles start beyond any request's tokens, which the kernels take as "nothing to do".
            n_tiles = -(-fixed.token_rows // PREFILL_TILE) + fixed.rows
            tile_seq = np.zeros(n_tiles, dtype=np.int32)
            tile_q0 = np.full(n_tiles, 1 << 30, dtype=np.int32)
            at = n_tiles
            for b in range(batch.B - 1, -1, -1):       # live tiles at the list's heavy end
                for q0 in range(-(-int(batch.count[b]) // PREFILL_TILE) - 1, -1, -1):
                    if batch.ctx_len[b] > 0:
                        at -= 1
                        tile_seq[at], tile_q0[at] = b, q0 * PREFILL_TILE
            return ({"tile_seq": tile_seq, "tile_q0": tile_q0},
                    dict(n_tiles=n_tiles, tile_keys=(PREFILL_TILE, fixed.max_context), n_dec=0, max_ctx_dec=0))
        start, count, ctx_len = batch.start, batch.count, batch.ctx_len
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
            tile_seq = tile_q0 = none
            tile_keys = (0, 0)
        arrays = {"tile_seq": tile_seq, "tile_q0": tile_q0}
        if dec.size:
            arrays["dec"] = dec
        return arrays, dict(n_tiles=int(tile_seq.size), tile_keys=tile_keys, n_dec=int(dec.size),
                            max_ctx_dec=int(ctx_len[dec].max()) if dec.size else 0)


_WORK = AttentionWork()


@MIXERS.register("paged_attention")
class PagedAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[PartSpec] = None, window: int = 0, scale: Optional[float] = None,
                 own_kv: bool = True):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not split over {num_kv_heads} key/value heads")
        if head_dim % 16 or not 16 <= head_dim <= 256:
            raise ValueError(f"the attention kernels take head sizes that are multiples of 16 up to 256, not {head_dim}")
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.window = int(window)
        self.scale = 1.0 / math.sqrt(head_dim) if scale is None else float(scale)
        self.own_kv = own_kv
        self.position = POSITION_ENCODINGS.build(position) if position is not None else None
        if self.position is not None and self.position.rotary_dim > head_dim:
            raise ValueError("rotary width exceeds the head size")
        self.qkv_proj: Optional[torch.Tensor] = None
        self.o_proj: Optional[torch.Tensor] = None

    def weight_specs(self):
        q = WeightSource("q_proj.weight", (self.num_heads * self.head_dim, self.hidden_size))
        kv_shape = (self.num_kv_heads * self.head_dim, self.hidden_size)
        sources = (q, WeightSource("k_proj.weight", kv_shape), WeightSource("v_proj.weight", kv_shape)) \
            if self.own_kv else (q,)
        return [
            WeightSpec("qkv_proj", sources),
            WeightSpec("o_proj", (WeightSource("o_proj.weight", (self.hidden_size, self.num_heads * self.head_dim)),)),
        ]

    def children(self):
        return {"rotary.": self.position} if self.position is not None else {}

    def cache_spec(self):
        return PagedSpec.keys_and_values(self.num_kv_heads, self.head_dim, self.window)

    def step_planner(self):
        return _WORK

    # The launch shapes of the two attention kernels for a step, from the planner's host values
    # alone (no device work: a test can check them against the kernels' index ranges).
    def prefill_launch(self, meta: dict, dtype: torch.dtype, page_size: int) -> Optional[dict]:
        """For the tiles of requests that bring several tokens: in how many runs every tile's keys
        are cut, whether workgroups pair a light tile with a heavy one, and the floats of the
        workspaces the runs' partial results need.  None: no tiles."""
        n_tiles = meta["n_tiles"]
        if not n_tiles:
            return None
        # Tiles come in rising order of the keys they see; when the first sees less than half
        # of what the last does, a workgroup may take one from each end.
        few, many = (min(k, self.window + 64) if self.window else k for k in meta["tile_keys"])
        # few new tokens over many keys: the keys in runs, for workgroups of their own
        parts = ops.attn_prefill_plan(n_tiles, many, self.num_heads, self.num_kv_heads, self.head_dim, dtype, page_size)
        n = n_tiles * PREFILL_TILE * self.num_heads * parts if parts > 1 else 0
        return dict(n_tiles=n_tiles, parts=parts, pair=2 * few <= many, part_o=n * self.head_dim, part_ml=n * 2)

    def decode_launch(self, meta: dict) -> Optional[dict]:
        """For the requests that bring one token: keys per workgroup, the most partitions a
        request can have, and the floats of the partitions' workspaces.  None: no such request."""
        n_dec, max_ctx = meta["n_dec"], meta["max_ctx_dec"]
        if not n_dec:
            return None
        part = ops.attn_decode_plan(n_dec, max_ctx, self.num_heads, self.num_kv_heads, self.head_dim)
        max_parts = max(1, (max_ctx + part - 1) // part)
        n = n_dec * self.num_heads * max_parts
        return dict(n_dec=n_dec, part_keys=part, max_parts=max_parts, part_o=n * self.head_dim, part_ml=n * 2)

    takes_pending_norm = True   # x may be an ops.PendingNorm: the q/k/v product norms on its way in

    def forward(self, ctx: StepContext, x, cache: LayerCache):
        if cache.writes != self.own_kv:
            raise RuntimeError("a mixer with its own keys must write the cache, one without must not")
        g = cache.group
        table = self.position.table if self.position is not None else None
        qkv = ops.linear_rope_kv(x, self.qkv_proj, ctx.positions, table, g.slot_mapping, cache.k, cache.v,
                                 num_heads=self.num_heads, num_kv_heads=self.num_kv_heads, head_dim=self.head_dim,
                                 page_size=g.page_size, has_kv=self.own_kv)
        out = torch.empty((ctx.T, self.num_heads * self.head_dim), dtype=ctx.dtype, device=qkv.device)
        common = dict(num_heads=self.num_heads, num_kv_heads=self.num_kv_heads, head_dim=self.head_dim,
                      window=self.window, scale=self.scale)
        work = ctx.plans[AttentionWork.key]
        pre = self.prefill_launch(work.meta, ctx.dtype, g.page_size)
        if pre is not None:
            part_o = part_ml = None
            if pre["parts"] > 1:
                part_o = ctx.scratch("attn_part_o", pre["part_o"])
                part_ml = ctx.scratch("attn_part_ml", pre["part_ml"])
            ops.attn_prefill(qkv, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.ctx_len,
                             work.arrays["tile_seq"], work.arrays["tile_q0"], pre["n_tiles"], pair=pre["pair"],
                             parts=pre["parts"], part_o=part_o, part_ml=part_ml, **common)
        dec = self.decode_launch(work.meta)
        if dec is not None:
            part_o = ctx.scratch("attn_part_o", dec["part_o"])
            part_ml = ctx.scratch("attn_part_ml", dec["part_ml"])
            ops.attn_decode(qkv, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.ctx_len,
                            work.arrays.get("dec"), dec["n_dec"], part_o, part_ml, dec["max_parts"], dec["part_keys"],
                            **common)
        return ops.linear(out, self.o_proj, out_dtype=ctx.dtype, may_split=True, pending=True)
