"""Chooses the next token of every row of logits, on the device.

What is computed is the reference's sample_next_tokens
(python/lyapunov_engine/engine/sampling.py:15-72); it runs there row by row with
a host round trip per row (``.item()``), here as one kernel launch for the
batch and one copy of the chosen tokens back.

The uniform number behind a draw comes from (engine seed, request seed, index of
the output token) through a counter-based generator, so it is the same whatever
else is in the batch, and the same again after a preemption.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .params import SamplingParams

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform(seed: int, stream: int, index: int) -> float:
    """A number in [0, 1) fixed by its three coordinates."""
    z = _splitmix64(seed & _MASK)
    z = _splitmix64(z ^ (stream & _MASK))
    z = _splitmix64(z ^ (index & _MASK))
    return (z >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, device, seed: int = 0):
        self.device = torch.device(device)
        self.seed = seed

    def sample(self, logits: torch.Tensor, params: list, streams: list, indices: list) -> list:
        """logits [R, vocab] float on the device; one SamplingParams, stream id
        and output index per row.  Returns R token ids."""
        R = logits.shape[0]
        if not (len(params) == len(streams) == len(indices) == R):
            raise ValueError("one set of sampling parameters per row of logits")
        host = torch.empty((4, R), dtype=torch.float32)
        for r, (p, s, i) in enumerate(zip(params, streams, indices)):
            host[0, r] = p.temperature
            host[1, r] = p.top_p
            host[2, r] = uniform(self.seed, s, i)
            host[3, r] = 0.0
        top_k = torch.tensor([p.top_k for p in params], dtype=torch.int32)
        dev = host.to(self.device)
        out = torch.empty(R, dtype=torch.int32, device=self.device)
        ops.sample(logits, dev[0], top_k.to(self.device), dev[1], dev[2], out)
        return out.cpu().tolist()


__all__ = ["Sampler", "SamplingParams", "uniform"]
