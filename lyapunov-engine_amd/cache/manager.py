"""The cache manager as Python sees it, and the device memory it hands out
numbers for.

``CacheManager`` wraps the C++ class of csrc/runtime/cache_manager.hpp (pages in
groups, block tables, windows, state slots; after the reference's
BlockSpaceManager, csrc/engine/block_manager.cpp:7-101).  ``CachePools`` holds
the tensors: per group, for every cache buffer of the group, the tensors its
mixers' ``PagedSpec`` names, and per stateful buffer one tensor of slots.  The
reference allocates two zero tensors [num_blocks, nkv, block_size, head_dim] per
layer (python/lyapunov_engine/engine/llm_engine.py:143-158); the layout here is
the mixer's choice (attention: keys as there, values
[num_blocks, nkv, head_dim, block_size], which its kernels read).
"""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_int32, c_int64
from dataclasses import dataclass

import torch

from . import runtime_lib


class CacheError(RuntimeError):
    pass


@dataclass(frozen=True)
class GroupConfig:
    num_pages: int
    page_size: int = 16
    window: int = 0


class CacheManager:
    def __init__(self, groups: list, num_state_slots: int):
        self._lib = runtime_lib.lib()
        self.groups = [g if isinstance(g, GroupConfig) else GroupConfig(*g) for g in groups]
        n = len(self.groups)
        arr = lambda vals: (c_int * n)(*vals)
        self._h = self._lib.lyp_cache_create(n, arr([g.num_pages for g in self.groups]),
                                             arr([g.page_size for g in self.groups]),
                                             arr([g.window for g in self.groups]), num_state_slots)
        if not self._h:
            raise CacheError(runtime_lib.last_error())
        self.num_state_slots = num_state_slots
        self._buf = (c_int32 * 64)()

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.lyp_cache_destroy(h)

    @property
    def handle(self):
        return self._h

    def _rc(self, rc: int) -> int:
        if rc < 0:
            raise CacheError(runtime_lib.last_error())
        return rc

    def add(self, seq_id: int) -> int:
        return self._rc(self._lib.lyp_cache_add(self._h, seq_id))

    def has(self, seq_id: int) -> bool:
        return bool(self._lib.lyp_cache_has(self._h, seq_id))

    def length(self, seq_id: int) -> int:
        return self._rc(self._lib.lyp_cache_length(self._h, seq_id))

    def capacity(self, seq_id: int) -> int:
        return self._rc(self._lib.lyp_cache_capacity(self._h, seq_id))

    def max_length(self, seq_id: int) -> int:
        return self._rc(self._lib.lyp_cache_max_length(self._h, seq_id))

    def can_extend(self, seq_id: int, new_len: int) -> bool:
        return bool(self._rc(self._lib.lyp_cache_can_extend(self._h, seq_id, new_len)))

    def extend(self, seq_id: int, new_len: int) -> None:
        self._rc(self._lib.lyp_cache_extend(self._h, seq_id, new_len))

    def commit(self, seq_id: int, new_len: int) -> None:
        self._rc(self._lib.lyp_cache_commit(self._h, seq_id, new_len))

    def free(self, seq_id: int) -> None:
        self._rc(self._lib.lyp_cache_free(self._h, seq_id))

    def reset(self) -> None:
        self._rc(self._lib.lyp_cache_reset(self._h))

    def num_free_pages(self, group: int = 0) -> int:
        return self._rc(self._lib.lyp_cache_num_free_pages(self._h, group))

    def num_free_slots(self) -> int:
        return self._lib.lyp_cache_num_free_slots(self._h)

    def num_requests(self) -> int:
        return self._lib.lyp_cache_num_requests(self._h)

    def state_slot(self, seq_id: int) -> int:
        return self._rc(self._lib.lyp_cache_state_slot(self._h, seq_id))

    def table(self, seq_id: int, group: int = 0) -> list:
        n = self._rc(self._lib.lyp_cache_table(self._h, seq_id, group, self._buf, len(self._buf)))
        if n > len(self._buf):
            self._buf = (c_int32 * (2 * n))()
            n = self._rc(self._lib.lyp_cache_table(self._h, seq_id, group, self._buf, len(self._buf)))
        return list(self._buf[:n])

    def export(self, seq_ids, group: int, tables, slots=None) -> None:
        """Block tables (and state slots) of several requests at once, written
        into int32 numpy arrays: row b of ``tables`` gets the table of
        ``seq_ids[b]`` (an int64 numpy array), as far as it goes."""
        self._rc(self._lib.lyp_cache_export(self._h, seq_ids.ctypes.data, len(seq_ids), group, tables.ctypes.data,
                                            tables.shape[1], slots.ctypes.data if slots is not None else None))

    def step_tables(self, seq_ids, start, count, group: int, tables, slot_map, slots=None) -> None:
        """The tables of one step, checked and written into int32 numpy arrays.
        Request ``seq_ids[b]`` (int64) continues at ``start[b]`` with
        ``count[b]`` new tokens (int32): it must hold exactly ``start[b]``
        tokens and have pages for the new ones.  Row b of ``tables`` gets its
        block table (-1 past its end), ``slot_map`` the page slot of every new
        token in order, ``slots`` the state slots."""
        self._rc(self._lib.lyp_cache_step_tables(self._h, seq_ids.ctypes.data, start.ctypes.data, count.ctypes.data,
                                                 len(seq_ids), group, tables.ctypes.data, tables.shape[1],
                                                 slot_map.ctypes.data, slots.ctypes.data if slots is not None else None))

    def reserve(self, seq_ids, new_lens) -> bool:
        """Pages for positions < new_lens[b] of every request seq_ids[b] (numpy
        int64 / int32 arrays), all or none: False, and nothing taken, if a
        group lacks the pages."""
        return bool(self._rc(self._lib.lyp_cache_reserve(self._h, seq_ids.ctypes.data, new_lens.ctypes.data,
                                                         len(seq_ids))))

    def ref_count(self, group: int, page: int) -> int:
        return self._rc(self._lib.lyp_cache_ref_count(self._h, group, page))

    def check(self) -> None:
        """Raise if an invariant is broken (a page lost, held twice, ...)."""
        if self._lib.lyp_cache_check(self._h) != 0:
            raise CacheError(runtime_lib.last_error())

    def counters(self) -> dict:
        out = (c_int64 * 4)()
        self._lib.lyp_cache_counters(self._h, out)
        return dict(pages_taken=out[0], pages_returned=out[1], window_returns=out[2], high_water=out[3])


class CachePools:
    """Device memory behind the page and slot numbers.

    ``paged[g]`` maps the names of group g's page tensors (its ``PagedSpec``:
    what the group's mixers keep per token, in the layout they chose) to
    tensors [buffers, pages, *page shape]; ``index[cache_id]`` says where a
    buffer lives; ``state[cache_id]`` is the slot tensor of a stateful buffer
    (its last slot belongs to no request: rows that are only padding use it).
    Everything starts at zero: a page that was never written must not hold a
    NaN pattern.
    """

    def __init__(self, layout, group_configs: list, num_state_slots: int, dtype: torch.dtype, device):
        if len(group_configs) != len(layout.groups):
            raise CacheError(f"{len(layout.groups)} cache groups need as many pool configurations")
        self.paged = []
        self.index = {}
        for g, (gl, gc) in enumerate(zip(layout.groups, group_configs)):
            nb = len(gl.buffers)
            self.paged.append({t.name: torch.zeros((nb, gc.num_pages) + t.page_shape(gc.page_size),
                                                   dtype=t.dtype or dtype, device=device) for t in gl.spec.tensors})
            for i, cache_id in enumerate(gl.buffers):
                self.index[cache_id] = (g, i)
        # one slot more than requests can hold: the padded rows of a recorded step are pointed at it
        self.state = {cid: torch.zeros((num_state_slots + 1,) + tuple(st.shape), dtype=st.dtype, device=device)
                      for cid, st in layout.states.items()}

    def buffer(self, cache_id: int):
        """-> (group, {page tensor name: [pages, *page shape]}) of one cache buffer."""
        g, i = self.index[cache_id]
        return g, {name: t[i] for name, t in self.paged[g].items()}

    def bytes(self) -> int:
        total = sum(t.numel() * t.element_size() for group in self.paged for t in group.values())
        return total + sum(s.numel() * s.element_size() for s in self.state.values())
