"""Rotary position encoding: the table of cosines and sines per position.

Frequencies and angles as the reference computes them
(python/lyapunov_engine/models/llama.py:180-194): inv_freq_i = theta^(-2i/d) in
32-bit, angle = position * inv_freq in 32-bit, one cosine and one sine per pair
(i, i + d/2).  The table's layout is the reference kernel's
(csrc/include/kernels/fused_rope.cuh:19, tests/test_fused_rope.py:13-24):
[max_position, d] with d/2 cosines followed by d/2 sines.  It is indexed with
each token's absolute position; the reference rebuilds it from 0 for every call
(llama.py:206-207), which gives a decoded token position 0.

The "llama3" frequency scaling is not in the reference.  By wavelength
2*pi/inv_freq against the original context length L: shorter than L/high stays;
longer than L/low is divided by ``factor``; in between the two are blended with
s = (L/wavelength - low) / (high - low): (1 - s) * inv_freq/factor + s * inv_freq.
"""
from __future__ import annotations

import math
import weakref
from typing import Optional

import torch

from ..config.registry import POSITION_ENCODINGS
from .base import PositionEncoding


def rotary_inv_freq(dim: int, theta: float, scaling: Optional[dict] = None) -> torch.Tensor:
    inv_freq = 1.0 / (theta ** (torch.arange(0, dim, 2).float() / dim))
    if not scaling or scaling.get("rope_type", "default") == "default":
        return inv_freq
    if scaling["rope_type"] != "llama3":
        raise ValueError(f"rotary scaling {scaling['rope_type']!r} is not implemented")
    factor = float(scaling["factor"])
    low = float(scaling["low_freq_factor"])
    high = float(scaling["high_freq_factor"])
    orig = float(scaling["original_max_position_embeddings"])
    wavelen = 2.0 * math.pi / inv_freq
    scaled = torch.where(wavelen > orig / low, inv_freq / factor, inv_freq)
    smooth = (orig / wavelen - low) / (high - low)
    blended = (1.0 - smooth) * inv_freq / factor + smooth * inv_freq
    medium = (wavelen >= orig / high) & (wavelen <= orig / low)
    return torch.where(medium, blended, scaled)


# Tables in use, by what fixes their contents: parts with equal parameters (the
# layers of a model, as a rule) share one tensor.  A table goes when the last
# part that uses it does.
_TABLES: "weakref.WeakValueDictionary" = weakref.WeakValueDictionary()


@POSITION_ENCODINGS.register("rope")
class RotaryEncoding(PositionEncoding):
    def __init__(self, dim: int, theta: float, max_position: int, scaling: Optional[dict] = None):
        if dim % 2:
            raise ValueError(f"rotary width {dim} must be even")
        self.rotary_dim = dim
        self.theta = float(theta)
        self.max_position = max_position
        self.positions = max_position      # rows of the table: max_position, or fewer (``limit_positions``)
        self.scaling = scaling
        self.table: Optional[torch.Tensor] = None

    def limit_positions(self, n: int) -> None:
        self.positions = max(1, min(self.max_position, int(n)))

    def build_table(self) -> torch.Tensor:
        inv_freq = rotary_inv_freq(self.rotary_dim, self.theta, self.scaling)
        angles = torch.outer(torch.arange(self.positions, dtype=torch.float32), inv_freq)
        return torch.cat((angles.cos(), angles.sin()), dim=-1).contiguous()

    def materialize(self, device, dtype):
        scaling = tuple(sorted(self.scaling.items())) if self.scaling else None
        key = (self.rotary_dim, self.theta, scaling, self.positions, str(torch.device(device)))
        table = _TABLES.get(key)
        if table is None:
            table = self.build_table().to(device)
            _TABLES[key] = table
        self.table = table


@POSITION_ENCODINGS.register("none")
class NoPositionEncoding(PositionEncoding):
    """No rotation: the mixer sees positions through the causal mask alone."""

    def __init__(self, **_):
        self.table = None
        self.rotary_dim = 0
