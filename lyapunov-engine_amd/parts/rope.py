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


@POSITION_ENCODINGS.register("rope")
class RotaryEncoding(PositionEncoding):
    def __init__(self, dim: int, theta: float, max_position: int, scaling: Optional[dict] = None):
        if dim % 2:
            raise ValueError(f"rotary width {dim} must be even")
        self.rotary_dim = dim
        self.theta = float(theta)
        self.max_position = max_position
        self.scaling = scaling
        self.table: Optional[torch.Tensor] = None

    def build_table(self) -> torch.Tensor:
        inv_freq = rotary_inv_freq(self.rotary_dim, self.theta, self.scaling)
        angles = torch.outer(torch.arange(self.max_position, dtype=torch.float32), inv_freq)
        return torch.cat((angles.cos(), angles.sin()), dim=-1).contiguous()

    def materialize(self, device, dtype):
        self.table = self.build_table().to(device)


@POSITION_ENCODINGS.register("none")
class NoPositionEncoding(PositionEncoding):
    """No rotation: the mixer sees positions through the causal mask alone."""

    def __init__(self, **_):
        self.table = None
        self.rotary_dim = 0
