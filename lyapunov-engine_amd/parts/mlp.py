"""SiLU-gated feed-forward.

down( silu(gate(x)) * up(x) ), no biases, with gate and up as one matrix whose
first rows are the gate (python/lyapunov_engine/models/llama.py:109-122;
models/weight_loader.py:155-163 builds cat([gate, up], dim=0); the activation is
python/lyapunov_engine/ops.py:72-73).
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import FEED_FORWARDS
from ..kernels import ops
from .base import FeedForward, StepContext, WeightSource, WeightSpec


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        # Rows of the fused matrix in tiles of 16 (eight gates, their eight ups) let a
        # decode step gate inside the product; widths that are no multiple of 8 keep
        # the plain order, gates first.
        self.interleave = 8 if intermediate_size % 8 == 0 else 0
        self.gate_up_proj: Optional[torch.Tensor] = None
        self.down_proj: Optional[torch.Tensor] = None

    def weight_specs(self):
        shape = (self.intermediate_size, self.hidden_size)
        return [
            WeightSpec("gate_up_proj", (WeightSource("gate_proj.weight", shape), WeightSource("up_proj.weight", shape)),
                       interleave=self.interleave),
            WeightSpec("down_proj", (WeightSource("down_proj.weight", (self.hidden_size, self.intermediate_size)),)),
        ]

    takes_pending_norm = True   # x may be an ops.PendingNorm: the gate/up product norms on its way in

    def forward(self, ctx: StepContext, x):
        act = ops.linear_swiglu(x, self.gate_up_proj, self.interleave)
        return ops.linear(act, self.down_proj, out_dtype=ctx.dtype, may_split=True, pending=True)
