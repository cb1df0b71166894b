"""Random weights from a configuration and a seed, as a model folder.

The reference has no such mode; its tests and benches take whatever torch's
module constructors draw (python/lyapunov_engine/models/llama.py:130-133,
172-177; benchmarks/bench_serving.py:34).  Here every tensor's values depend on
(seed, tensor name) alone, so they do not change with the order in which tensors
are made or with what else the model holds: matrices and the embedding are
normal(0, init_std), norm weights are 1 + normal(0, norm_init_std).
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Iterator, Optional

import torch

from ..config.registry import ARCHITECTURES, architecture_of
from ..models.decoder import build_model
from .safetensors_io import write_safetensors

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def _tensor_seed(seed: int, name: str) -> int:
    return int.from_bytes(hashlib.sha256(f"{seed}:{name}".encode()).digest()[:8], "little") & ((1 << 63) - 1)


def random_tensors(model, seed: int, dtype: torch.dtype, init_std: Optional[float] = None,
                   norm_init_std: Optional[float] = None, device="cpu") -> Iterator[tuple]:
    """(name, tensor) for every tensor the model expects.  On ``device="cpu"``
    (the mode that writes model folders) values are reproducible everywhere; on
    a GPU they come from that device's generator, which is faster for large
    models and only used where the values do not matter."""
    spec = model.spec
    std = spec.init_std if init_std is None else init_std
    nstd = spec.norm_init_std if norm_init_std is None else norm_init_std
    for name, (shape, init) in model.expected_tensors().items():
        gen = torch.Generator(device=device)
        gen.manual_seed(_tensor_seed(seed, name))
        t = torch.randn(shape, generator=gen, dtype=torch.float32, device=device)
        if init == "ones":
            t = 1.0 + t * nstd
        elif init == "normal":
            t = t * std
        else:
            raise ValueError(f"unknown init kind {init!r} for {name}")
        yield name, t.to(dtype)


def write_random_model(config, folder: str, seed: int, dtype: str = "bfloat16", init_std: Optional[float] = None,
                       norm_init_std: Optional[float] = None) -> str:
    """Write ``config.json`` and ``model.safetensors`` for a typed configuration
    (or a config dict).  Returns the folder."""
    if isinstance(config, dict):
        arch = architecture_of(config)
        config = arch.config_class.from_dict(config)
    else:
        arch = ARCHITECTURES.get(config.architectures[0])
    if dtype not in _STORE:
        raise ValueError(f"weights can be stored as {sorted(_STORE)}, not {dtype!r}")
    os.makedirs(folder, exist_ok=True)
    model = build_model(arch.to_spec(config))
    tensors = dict(random_tensors(model, seed, _STORE[dtype], init_std, norm_init_std))
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": seed})
    d = config.to_dict()
    d["torch_dtype"] = dtype
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(d, f, indent=2)
    return folder
