"""Per-request sampling options.

The five fields and their defaults are the reference's
(python/lyapunov_engine/engine/sampling.py:6-12; C++ mirror
csrc/include/engine/sequence.hpp:20-26).  ``seed`` is added: the reference draws
from torch's global generator (sampling.py:69), so a request's tokens depend on
what else runs; here each request has a stream of its own.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class SamplingParams:
    temperature: float = 1.0
    top_p: float = 1.0
    top_k: int = -1
    max_tokens: int = 128
    ignore_eos: bool = False
    seed: Optional[int] = None

    def __post_init__(self):
        if self.max_tokens <= 0:
            raise ValueError("max_tokens must be positive")
        if not 0.0 <= self.top_p <= 1.0:
            raise ValueError("top_p must lie in [0, 1]")

    @property
    def greedy(self) -> bool:
        # sampling.py:34: "temperature <= 0.0 or temperature < 1e-4"
        return self.temperature < 1e-4
