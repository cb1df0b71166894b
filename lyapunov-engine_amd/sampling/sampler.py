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
        self._cap = 0
        self._host = self._dev = self._out = None

    def _reserve(self, rows: int) -> None:
        if rows > self._cap:
            self._cap = max(rows, 2 * self._cap, 64)
            # rows of the parameter block: temperature, top_p, uniform, top_k (as int32 bits)
            self._host = torch.zeros((4, self._cap), dtype=torch.float32).pin_memory()
            self._dev = torch.zeros((4, self._cap), dtype=torch.float32, device=self.device)
            self._out = torch.zeros(self._cap, dtype=torch.int32, device=self.device)
            self._work = ops.sample_workspace(self._cap, self.device)
            self._greedy_on_device = True   # the device block is all zeros: temperature 0 everywhere

    def sample(self, logits: torch.Tensor, params: list, streams: list, indices: list) -> list:
        """logits [R, vocab] float on the device; one SamplingParams, stream id
        and output index per row.  Returns R token ids."""
        R = logits.shape[0]
        if not (len(params) == len(streams) == len(indices) == R):
            raise ValueError("one set of sampling parameters per row of logits")
        self._reserve(R)
        if all(p.temperature < 1e-4 for p in params):
            if not self._greedy_on_device:
                self._dev.zero_()
                self._greedy_on_device = True
        else:
            h = self._host
            hk = h[3].view(torch.int32)
            for r, (p, s, i) in enumerate(zip(params, streams, indices)):
                h[0, r] = p.temperature
                h[1, r] = p.top_p
                h[2, r] = uniform(self.seed, s, i)
                hk[r] = p.top_k
            self._dev[:, :R].copy_(h[:, :R], non_blocking=True)
            self._greedy_on_device = False
        d = self._dev
        out = self._out[:R]
        ops.sample(logits, d[0, :R], d[3, :R].view(torch.int32), d[1, :R], d[2, :R], out, self._work)
        return out.tolist()


__all__ = ["Sampler", "SamplingParams", "uniform"]
