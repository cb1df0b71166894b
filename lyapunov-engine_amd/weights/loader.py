"""Binds the tensors of a model folder to the parts of a model, by name.

The reference's loader (python/lyapunov_engine/models/weight_loader.py:74-171)
guards every name with ``if key in weights`` and so leaves a missing tensor at
its random initial value without a word; a wrong shape surfaces as a ``copy_``
error.  Here the model says which names and shapes it expects
(``DecoderModel.expected_tensors``), the files say what they hold, and any
difference (missing, unexpected, wrong shape) is reported in one error that
lists all of them.  As in the reference gate_proj and up_proj become one matrix
(:155-163); so do q_proj, k_proj and v_proj.

Precision: with the engine in bfloat16, floating tensors are kept in bfloat16,
except that a tensor the file stores in 32-bit stays in 32-bit; integer tensors
become int32.  With the engine in float32 every floating tensor becomes float32.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import load_config
from ..models.decoder import DecoderModel, build_model
from ..utils import log
from .safetensors_io import open_model_files


class WeightError(ValueError):
    pass


class TensorSource:
    """Where tensors come from: name -> shape, and name -> CPU tensor."""

    def shapes(self) -> dict:
        raise NotImplementedError

    def get(self, name: str) -> torch.Tensor:
        raise NotImplementedError


class FolderSource(TensorSource):
    def __init__(self, model_dir: str):
        self.files = open_model_files(model_dir)
        self.where = {}
        for f in self.files:  # later files overwrite earlier ones (models/weight_loader.py:53-56: update() in sorted file order)
            for name in f.names():
                self.where[name] = f

    def shapes(self):
        return {name: f.entries[name].shape for name, f in self.where.items()}

    def get(self, name):
        return self.where[name].tensor(name)


class DictSource(TensorSource):
    def __init__(self, tensors: dict):
        self.tensors = tensors

    def shapes(self):
        return {k: tuple(v.shape) for k, v in self.tensors.items()}

    def get(self, name):
        return self.tensors[name]


def check_tensors(model: DecoderModel, present: dict) -> None:
    expected = model.expected_tensors()
    missing = sorted(n for n in expected if n not in present)
    unexpected = sorted(n for n in present if n not in expected and not model.ignorable(n))
    wrong = sorted((n, tuple(present[n]), expected[n][0]) for n in expected
                   if n in present and tuple(present[n]) != tuple(expected[n][0]))
    if not (missing or unexpected or wrong):
        return
    lines = ["the model's tensors do not match its configuration:"]
    if missing:
        lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
    if wrong:
        lines.append(f"  wrong shape ({len(wrong)}): " +
                     ", ".join(f"{n} is {list(got)}, expected {list(want)}" for n, got, want in wrong))
    raise WeightError("\n".join(lines))


def kept_dtype(stored: torch.dtype, engine_dtype: torch.dtype) -> torch.dtype:
    if not stored.is_floating_point:
        return torch.int32
    if engine_dtype == torch.float32 or stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def load_weights(model: DecoderModel, source: TensorSource, dtype: torch.dtype, device,
                 max_positions: Optional[int] = None) -> DecoderModel:
    check_tensors(model, source.shapes())
    expected = model.expected_tensors()
    for name in sorted(n for n in source.shapes() if n not in expected):
        log.info(f"note: {name} is in the files and not used by this model (a separate head of a tied "
                 f"model, or a buffer the architecture declares ignorable); ignored")
    device = torch.device(device)
    for owner, ws in model.weight_table():
        pieces = [source.get(s.name) for s in ws.sources]
        kinds = {kept_dtype(p.dtype, dtype) for p in pieces}
        keep = torch.float32 if torch.float32 in kinds else kinds.pop()
        pieces = [p.to(device=device, dtype=keep, non_blocking=False) for p in pieces]
        t = pieces[0] if len(pieces) == 1 else torch.cat(pieces, dim=0)
        if ws.interleave:
            n, k = ws.interleave, len(pieces)
            rows = pieces[0].shape[0]
            if any(p.shape != pieces[0].shape for p in pieces) or rows % n:
                raise WeightError(f"{ws.attr}: rows of {[tuple(p.shape) for p in pieces]} cannot alternate in runs of {n}")
            t = t.view(k, rows // n, n, *t.shape[1:]).transpose(0, 1).reshape(t.shape)
        setattr(owner, ws.attr, t.contiguous())
    model.materialize(device, dtype, max_positions)
    return model


def load_model(model_dir: str, dtype: torch.dtype, device="cuda:0", source: Optional[TensorSource] = None,
               max_positions: Optional[int] = None):
    """config.json -> architecture -> model, with its tensors from the folder's
    safetensors files.  Returns (model, typed configuration).  ``max_positions``:
    see ``DecoderModel.materialize``; a function is called with the model as
    built (its parts and cache layout are known, its weights not yet loaded) and
    returns the number."""
    arch, cfg = load_config(model_dir)
    model = build_model(arch.to_spec(cfg))
    if callable(max_positions):
        max_positions = max_positions(model)
    load_weights(model, source or FolderSource(model_dir), dtype, device, max_positions)
    return model, cfg
