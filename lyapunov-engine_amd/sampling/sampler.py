"""Chooses the next token of every row of logits, on the device.

What is computed is the reference's sample_next_tokens
(python/lyapunov_engine/engine/sampling.py:15-72); it runs there row by row with
a host round trip per row (``.item()``), here as one launch for the batch
whose kernel writes the chosen tokens to the device (for a step that is started
before the host has them) and to pinned host memory (read behind an event).

The uniform number behind a draw comes from (engine seed, request seed, index of
the output token) through a counter-based generator, so it is the same whatever
else is in the batch, and the same again after a preemption.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..parts.base import Logits
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


class PendingSample:
    """Tokens that the device is still choosing: ``tokens`` is the device
    tensor they go to (usable by later work on the stream at once), ``result()``
    waits for the copy to the host and returns them as a list."""

    def __init__(self, tokens: torch.Tensor, host: torch.Tensor, event: torch.cuda.Event):
        self.tokens, self._host, self._event = tokens, host, event

    def result(self) -> list:
        self._event.synchronize()
        return self._host.tolist()


class Sampler:
    RING = 4   # sets of buffers in turn: a set is not touched again while its step may still be in flight

    def __init__(self, device, seed: int = 0):
        self.device = torch.device(device)
        self.seed = seed
        self._cap = 0
        self._turn = 0
        self._sets: list = []

    def _reserve(self, rows: int) -> None:
        if rows > self._cap:
            self._cap = max(rows, 2 * self._cap, 64)
            self._sets = []
            for _ in range(self.RING):
                # rows of the parameter block: temperature, top_p, uniform, top_k (as int32 bits)
                self._sets.append(dict(
                    host=torch.zeros((4, self._cap), dtype=torch.float32).pin_memory(),
                    out=torch.zeros(self._cap, dtype=torch.int32, device=self.device),
                    out_host=torch.zeros(self._cap, dtype=torch.int32).pin_memory(),
                    event=torch.cuda.Event()))
            self._dev = torch.zeros((4, self._cap), dtype=torch.float32, device=self.device)
            self._work = ops.sample_workspace(self._cap, self.device)
            self._greedy_on_device = True   # the device block is all zeros: temperature 0 everywhere

    def launch(self, logits, params: list, streams: list, indices: list) -> PendingSample:
        """``logits``: a step's ``Logits`` (values [R, vocab] float on the device,
        with the row maxima its head may have left), or just the tensor of
        values; one SamplingParams, stream id and output index per row.  Starts
        the choice of R token ids and their copy to the host; nothing waits here."""
        row_maxima = None
        if isinstance(logits, Logits):
            logits, row_maxima = logits.values, logits.row_maxima
        R = logits.shape[0]
        if not (len(params) == len(streams) == len(indices) == R):
            raise ValueError("one set of sampling parameters per row of logits")
        self._reserve(R)
        bufs = self._sets[self._turn]
        self._turn = (self._turn + 1) % self.RING
        if all(p.temperature < 1e-4 for p in params):
            if not self._greedy_on_device:
                self._dev.zero_()
                self._greedy_on_device = True
        else:
            h = bufs["host"]
            hk = h[3].view(torch.int32)
            for r, (p, s, i) in enumerate(zip(params, streams, indices)):
                h[0, r] = p.temperature
                h[1, r] = p.top_p
                h[2, r] = uniform(self.seed, s, i)
                hk[r] = p.top_k
            self._dev[:, :R].copy_(h[:, :R], non_blocking=True)
            self._greedy_on_device = False
        d = self._dev
        out = bufs["out"][:R]
        host = bufs["out_host"][:R]
        # the kernel writes the tokens to the pinned buffer itself: no copy after it
        ops.sample(logits, d[0, :R], d[3, :R].view(torch.int32), d[1, :R], d[2, :R], out, self._work, mirror=host,
                   row_maxima=row_maxima)
        bufs["event"].record()
        return PendingSample(out, host, bufs["event"])

    def sample(self, logits: torch.Tensor, params: list, streams: list, indices: list) -> list:
        """The same, waited for: R token ids."""
        return self.launch(logits, params, streams, indices).result()


__all__ = ["Sampler", "PendingSample", "SamplingParams", "uniform"]
