"""Run-time options of the engine.

Names and defaults follow the reference's EngineConfig
(python/lyapunov_engine/engine/llm_engine.py:18-38): ``num_blocks`` (alias
``num_gpu_blocks``) 1024, ``block_size`` 16, ``max_num_seqs`` 64,
``max_num_batched_tokens`` 2048, ``dtype``, ``device``.  Added: the model length,
the longest prompt portion per step, a seed, the graph, look-ahead and warm-up switches, and an override
of the end-of-sequence ids (the reference fixes 128001 in its scheduler,
csrc/include/engine/scheduler.hpp:16).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

_DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16, torch.bfloat16: torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "float": torch.float32, torch.float32: torch.float32,
}


def parse_dtype(dtype) -> torch.dtype:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}") from None


@dataclass
class EngineConfig:
    model_config: object = None
    num_blocks: int = 1024
    num_gpu_blocks: Optional[int] = None
    block_size: int = 16
    cache_groups: Optional[tuple] = None    # per cache group of the model (pages, page size) where they differ; see EngineCore
    max_num_seqs: int = 64
    max_num_batched_tokens: int = 2048
    dtype: object = "bfloat16"
    device: str = "cuda:0"
    max_model_len: Optional[int] = None     # default: the model's max_position_embeddings
    max_chunk: int = 0                      # longest prompt portion in a step; 0: the token budget decides
    seed: int = 0
    enable_graphs: bool = True              # replay pure-decode steps from captured HIP graphs
    lookahead: bool = True                  # start the next decode step before this one's tokens reach the host
    eos_token_ids: Optional[tuple] = None   # default: the model's
    warmup: bool = True                     # run one full step at start-up: libraries loaded, GEMM algorithms chosen by measurement

    def __post_init__(self):
        if self.num_gpu_blocks is not None:
            self.num_blocks = self.num_gpu_blocks
        self.dtype = parse_dtype(self.dtype)
        for name in ("num_blocks", "block_size", "max_num_seqs", "max_num_batched_tokens"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")
        if self.max_chunk < 0:
            raise ValueError("max_chunk must be 0 (off) or positive")
