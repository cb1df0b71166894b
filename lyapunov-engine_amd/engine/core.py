"""Model, cache manager, device pools and step function as one object; what the
generating engine and the trace replay both stand on."""
from __future__ import annotations

from typing import Optional

import torch

from ..cache.manager import CacheManager, CachePools, GroupConfig
from ..config.engine_config import parse_dtype
from ..models.decoder import DecoderModel
from ..weights.loader import TensorSource, load_model
from .runner import ModelRunner, StepEntry


class EngineCore:
    def __init__(self, model: DecoderModel, model_config, *, dtype, device="cuda:0", num_blocks: int,
                 block_size: int = 16, num_state_slots: int = 64, cache_groups: Optional[list] = None):
        """``cache_groups``: (pages, page size) for each of the model's cache
        groups in turn (``model.cache_layout().groups``: layers whose keys and
        values have one shape and one window share a group), where they are to
        differ from ``num_blocks`` and ``block_size``; None in place of a pair
        keeps those.  A group of windowed layers needs far fewer pages than one
        that keeps every key."""
        from ..kernels import ops

        ops.require_gpu()   # no CPU path: say so before anything is allocated
        self.model, self.model_config = model, model_config
        self.dtype, self.device = parse_dtype(dtype), torch.device(device)
        self.block_size = block_size
        layout = model.cache_layout()
        sizes = self.group_sizes(layout, num_blocks, block_size, cache_groups)
        groups = [GroupConfig(pages, size, gl.spec.window) for (pages, size), gl in zip(sizes, layout.groups)]
        # A model without keys and values (state only) still gets a group, so
        # that requests have a length and the manager one code path.
        self.cache = CacheManager(groups or [GroupConfig(num_blocks, block_size, 0)], num_state_slots)
        self.pools = CachePools(layout, groups, num_state_slots, self.dtype, self.device)
        self.runner = ModelRunner(model, self.cache, self.pools, self.dtype, self.device)

    @staticmethod
    def group_sizes(layout, num_blocks: int, block_size: int, cache_groups: Optional[list]) -> list:
        """(pages, page size) of every cache group of ``layout``, in order."""
        sizes = list(cache_groups or [])
        if len(sizes) > len(layout.groups):
            raise ValueError(f"cache_groups names {len(sizes)} groups, the model has {len(layout.groups)}")
        sizes += [None] * (len(layout.groups) - len(sizes))
        return [(num_blocks, block_size) if s is None else (int(s[0]), int(s[1])) for s in sizes]

    @staticmethod
    def reach(model: DecoderModel, num_blocks: int, block_size: int, cache_groups: Optional[list],
              max_model_len: Optional[int]) -> int:
        """The positions a request of this engine can ever reach: its model
        length, and the pool of every cache group that keeps all of a request's
        tokens (a group of windowed layers gives pages back as the window
        passes, so its pool bounds the window and the step's portion, not the
        request; a model that keeps everything in windows or in state is bound
        by the model length alone)."""
        layout = model.cache_layout()
        sizes = EngineCore.group_sizes(layout, num_blocks, block_size, cache_groups)
        bounds = [pages * size for (pages, size), gl in zip(sizes, layout.groups) if gl.spec.window == 0]
        reach = min(bounds) if bounds else model.spec.max_position
        return min(reach, int(max_model_len)) if max_model_len else reach

    @classmethod
    def from_folder(cls, model_dir: str, *, dtype, device="cuda:0", source: Optional[TensorSource] = None,
                    max_model_len: Optional[int] = None, **kw):
        """``max_model_len``: no request will be longer; with the pools of the
        cache groups that keep every token (see ``reach``) it bounds the
        positions the model is set up for (the rows of its position tables)."""
        def reach(model):
            return cls.reach(model, kw["num_blocks"], kw.get("block_size", 16), kw.get("cache_groups"), max_model_len)

        model, cfg = load_model(model_dir, parse_dtype(dtype), device, source=source, max_positions=reach)
        return cls(model, cfg, dtype=dtype, device=device, **kw)

    def step(self, entries: list):
        return self.runner.step(entries)


__all__ = ["EngineCore", "StepEntry"]
