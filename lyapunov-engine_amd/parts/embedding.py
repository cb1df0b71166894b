"""The two ends of the decoder: token embedding and output head.

The reference's LlamaForCausalLM holds ``model.embed_tokens`` (an nn.Embedding)
and ``lm_head`` (an nn.Linear without bias) and, where the head's tensor is
missing, copies the embedding into it
(python/lyapunov_engine/models/llama.py:172-177, 205, 224;
models/weight_loader.py:102-109).  Here the residual stream is float from the
first value on, logits are float, and a tied head uses the embedding's matrix
itself.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import EMBEDDINGS, HEADS
from ..kernels import ops
from .base import Embedding, Head, Logits, StepContext, WeightSource, WeightSpec


@EMBEDDINGS.register("lookup")
class TokenEmbedding(Embedding):
    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.weight: Optional[torch.Tensor] = None

    def weight_specs(self):
        return [WeightSpec("weight", (WeightSource("weight", (self.vocab_size, self.hidden_size)),))]

    def forward(self, ctx: StepContext, token_ids: torch.Tensor) -> torch.Tensor:
        h = torch.empty((token_ids.numel(), self.hidden_size), dtype=torch.float32, device=ctx.device)
        return ops.embedding(token_ids, self.weight, h)


@HEADS.register("linear")
class LinearHead(Head):
    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.weight: Optional[torch.Tensor] = None
        self._tied_to: Optional[Embedding] = None

    def tie(self, embedding: Embedding) -> None:
        self._tied_to = embedding

    def weight_specs(self):
        if self._tied_to is not None:
            return []
        return [WeightSpec("weight", (WeightSource("weight", (self.vocab_size, self.hidden_size)),))]

    def materialize(self, device, dtype):
        if self._tied_to is not None:
            self.weight = self._tied_to.weight      # one matrix, two uses

    def forward(self, ctx: StepContext, x: torch.Tensor) -> Logits:
        return Logits(*ops.lm_head(x, self.weight))
