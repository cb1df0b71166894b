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

import torch

from ..config.registry import MIXERS, POSITION_ENCODINGS
from ..config.specs import PartSpec
from ..kernels import ops
from .base import KVCacheSpec, LayerCache, Mixer, StepContext, WeightSource, WeightSpec


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
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window)

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
        if ctx.n_tiles:
            # Tiles come in rising order of the keys they see; when the first sees less than half
            # of what the last does, a workgroup may take one from each end.
            few, many = (min(k, self.window + 64) if self.window else k for k in ctx.tile_keys)
            # few new tokens over many keys: the keys in runs, for workgroups of their own
            parts = ops.attn_prefill_plan(ctx.n_tiles, many, self.num_heads, self.num_kv_heads, self.head_dim,
                                          ctx.dtype, g.page_size)
            part_o = part_ml = None
            if parts > 1:
                n = ctx.n_tiles * 64 * self.num_heads * parts
                part_o = ctx.scratch("attn_part_o", n * self.head_dim)
                part_ml = ctx.scratch("attn_part_ml", n * 2)
            ops.attn_prefill(qkv, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.ctx_len, ctx.tile_seq,
                             ctx.tile_q0, ctx.n_tiles, pair=2 * few <= many, parts=parts, part_o=part_o,
                             part_ml=part_ml, **common)
        if ctx.n_dec:
            part = ops.attn_decode_plan(ctx.n_dec, ctx.max_ctx_dec, self.num_heads, self.num_kv_heads, self.head_dim)
            max_parts = max(1, (ctx.max_ctx_dec + part - 1) // part)
            n = ctx.n_dec * self.num_heads * max_parts
            part_o = ctx.scratch("attn_part_o", n * self.head_dim)
            part_ml = ctx.scratch("attn_part_ml", n * 2)
            ops.attn_decode(qkv, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.ctx_len, ctx.dec_seqs,
                            ctx.n_dec, part_o, part_ml, max_parts, part, **common)
        return ops.linear(out, self.o_proj, out_dtype=ctx.dtype, may_split=True, pending=True)
