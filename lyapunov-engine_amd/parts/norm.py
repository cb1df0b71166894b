"""RMSNorm over the hidden dimension, fused with the residual add.

x * rsqrt(mean(x^2) + eps) * weight, all in 32-bit, as the reference's eager
path (python/lyapunov_engine/ops.py:49-50) and kernel
(csrc/kernels/fused_rmsnorm_swiglu.cu:83-84, 96-101).  The reference's model adds
the residual separately (models/llama.py:158, 164); here the add rides in the
norm that follows it, on a float residual stream.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import NORMS
from ..kernels import ops
from .base import Norm, StepContext, WeightSource, WeightSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    def __init__(self, size: int, eps: float):
        self.size = size
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def weight_specs(self):
        return [WeightSpec("weight", (WeightSource("weight", (self.size,)),), init="ones")]

    # With ``lazy`` the norm may add the delta and hand the rows on as an
    # ops.PendingNorm for the consumer's kernel to norm on its way in.
    can_defer = True

    def forward(self, ctx: StepContext, h, delta=None, rows=None, lazy=False):
        if lazy and rows is None:
            pending, delta = ops.rmsnorm_pending(h, self.weight, self.eps, ctx.dtype, delta)
            if pending is not None:
                return pending
        n = h.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.size), dtype=ctx.dtype, device=h.device)
        return ops.rmsnorm(h, self.weight, self.eps, out, delta=delta, rows=rows)
