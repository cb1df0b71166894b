"""Trace replay: feed given token ids through the model step by step and keep
the logits.  Nothing is sampled and nothing is scheduled; pages are taken from
the same cache manager, and the steps run through the same step function, as in
generation.  The reference has nothing like it (its nearest relative,
benchmarks/bench_serving.py:36-77, only times ``engine.step()``).

A step is a dict ``{"step": n, "entries": [{"id", "tokens", "want"}], "end": [ids]}``.
"""
from __future__ import annotations

from typing import Optional

import numpy as np

from .core import EngineCore, StepEntry

MAX_LIVE_REQUESTS = 8


class TraceReplayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, block_size: int = 16, device: str = "cuda:0",
                 cache_groups=None):
        num_blocks = max(1, -(-max_tokens // block_size))
        self.core = EngineCore.from_folder(model_dir, dtype=dtype, device=device, num_blocks=num_blocks,
                                           block_size=block_size, num_state_slots=MAX_LIVE_REQUESTS,
                                           cache_groups=cache_groups)
        self._ids: dict = {}
        self._next_id = 0

    def _seq(self, name) -> int:
        if name not in self._ids:
            self._ids[name] = self._next_id
            self._next_id += 1
            self.core.cache.add(self._ids[name])
        return self._ids[name]

    def run(self, step: dict) -> Optional[np.ndarray]:
        """Run one step; returns float32 logits [wanted, vocab] or None."""
        cache = self.core.cache
        entries = []
        for e in step.get("entries", []):
            tokens = [int(t) for t in e["tokens"]]
            if not tokens:
                continue
            seq = self._seq(e["id"])
            start = cache.length(seq)
            cache.extend(seq, start + len(tokens))
            entries.append(StepEntry(seq, tokens, start, [int(w) for w in e.get("want", [])]))
        logits = self.core.step(entries) if entries else None
        for e in entries:
            cache.commit(e.seq_id, e.start + len(e.tokens))
        for name in step.get("end", []):
            if name in self._ids:
                cache.free(self._ids.pop(name))
        if logits is None:
            return None
        return logits.detach().to("cpu").numpy().astype("<f4", copy=False)
