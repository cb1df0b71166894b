"""Typed configuration of the Llama decoder, read from config.json.

The reference's LlamaConfig has ten fields with the sizes of Llama 3.2 1B as
defaults, filled by ``cfg_dict.get(key, default)``
(python/lyapunov_engine/models/llama.py:9-20, models/weight_loader.py:10-38), and
knows neither ``rope_scaling`` nor ``tie_word_embeddings`` nor ``architectures``.
Here every size and constant comes from the file: a missing size is an error,
not a silent 1B default.  Keys whose absence has a meaning by the convention of
the file format have that meaning (``num_key_value_heads`` -> as many as query
heads, ``head_dim`` -> hidden_size // num_attention_heads as in
weight_loader.py:30-34, ``rope_scaling`` -> none, ``tie_word_embeddings`` ->
false, ``rope_theta`` -> 10000.0: files of the format's first generation do not
name the base and mean that one; the reference's fallback is the 1B model's
500000.0, weight_loader.py:37, which would rotate such a model's heads wrongly).
"""
from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass, field
from typing import Any, Optional


class ConfigError(ValueError):
    pass


@dataclass(frozen=True)
class RopeScaling:
    """The ``rope_scaling`` object of config.json.  ``llama3`` rescales the
    rotation frequencies by wavelength; ``default`` leaves them alone."""

    rope_type: str = "default"
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position_embeddings: int = 8192

    @staticmethod
    def from_dict(d: Optional[dict]) -> Optional["RopeScaling"]:
        if d is None:
            return None
        if not isinstance(d, dict):
            raise ConfigError(f"rope_scaling must be an object or null, got {type(d).__name__}")
        kind = d.get("rope_type", d.get("type", "default"))
        if kind == "default":
            return None
        if kind != "llama3":
            raise ConfigError(f"rope_scaling type {kind!r} is not implemented (known: 'llama3', 'default')")
        missing = [k for k in ("factor", "low_freq_factor", "high_freq_factor", "original_max_position_embeddings")
                   if k not in d]
        if missing:
            raise ConfigError(f"rope_scaling of type 'llama3' lacks {missing}")
        rs = RopeScaling("llama3", float(d["factor"]), float(d["low_freq_factor"]), float(d["high_freq_factor"]),
                         int(d["original_max_position_embeddings"]))
        if rs.factor <= 0 or rs.high_freq_factor <= rs.low_freq_factor or rs.original_max_position_embeddings <= 0:
            raise ConfigError(f"rope_scaling has impossible values: {d}")
        return rs

    def to_dict(self) -> dict:
        return {
            "rope_type": self.rope_type,
            "factor": self.factor,
            "low_freq_factor": self.low_freq_factor,
            "high_freq_factor": self.high_freq_factor,
            "original_max_position_embeddings": self.original_max_position_embeddings,
        }


_REQUIRED = (
    "vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
    "max_position_embeddings", "rms_norm_eps",
)
ROPE_THETA_CONVENTION = 10000.0   # what a config.json of this format means when it does not name rope_theta


def _as_id_tuple(v: Any) -> tuple:
    if v is None:
        return ()
    if isinstance(v, (list, tuple)):
        return tuple(int(x) for x in v)
    return (int(v),)


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: Optional[RopeScaling] = None
    tie_word_embeddings: bool = False
    architectures: tuple = ("LlamaForCausalLM",)
    eos_token_id: tuple = ()
    bos_token_id: Optional[int] = None
    torch_dtype: Optional[str] = None
    extra: dict = field(default_factory=dict, compare=False, repr=False)

    # ------------------------------------------------------------------ parsing
    @classmethod
    def from_dict(cls, d: dict) -> "LlamaConfig":
        missing = [k for k in _REQUIRED if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks {missing}")
        if d.get("attention_bias") or d.get("mlp_bias"):
            raise ConfigError("projections with a bias (attention_bias / mlp_bias) are not implemented")
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act {act!r} is not implemented (the feed-forward here is SiLU-gated)")
        nh = int(d["num_attention_heads"])
        hidden = int(d["hidden_size"])
        head_dim = d.get("head_dim")
        if head_dim is None:
            if nh <= 0 or hidden % nh:
                raise ConfigError(f"hidden_size {hidden} does not split over {nh} heads and no head_dim is given")
            head_dim = hidden // nh
        known = set(_REQUIRED) | {
            "rope_theta", "num_key_value_heads", "head_dim", "rope_scaling", "tie_word_embeddings", "architectures",
            "eos_token_id", "bos_token_id", "torch_dtype", "attention_bias", "mlp_bias", "hidden_act",
        }
        nkv = d.get("num_key_value_heads")
        cfg = cls(
            vocab_size=int(d["vocab_size"]),
            hidden_size=hidden,
            intermediate_size=int(d["intermediate_size"]),
            num_hidden_layers=int(d["num_hidden_layers"]),
            num_attention_heads=nh,
            num_key_value_heads=int(nkv) if nkv is not None else nh,
            head_dim=int(head_dim),
            max_position_embeddings=int(d["max_position_embeddings"]),
            rms_norm_eps=float(d["rms_norm_eps"]),
            rope_theta=float(d.get("rope_theta", ROPE_THETA_CONVENTION)),
            rope_scaling=RopeScaling.from_dict(d.get("rope_scaling")),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            architectures=tuple(d.get("architectures") or ("LlamaForCausalLM",)),
            eos_token_id=_as_id_tuple(d.get("eos_token_id")),
            bos_token_id=None if d.get("bos_token_id") is None else int(d["bos_token_id"]),
            torch_dtype=d.get("torch_dtype"),
            extra={k: v for k, v in d.items() if k not in known},
        )
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str) -> "LlamaConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path, "r", encoding="utf-8") as f:
            return cls.from_dict(json.load(f))

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"{self.num_attention_heads} query heads do not split over "
                              f"{self.num_key_value_heads} key/value heads")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even for the rotary encoding")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta}")
        for t in self.eos_token_id:
            if not 0 <= t < self.vocab_size:
                raise ConfigError(f"eos_token_id {t} is outside the vocabulary of {self.vocab_size}")

    # ------------------------------------------------------------------ writing
    def to_dict(self) -> dict:
        d = {
            "architectures": list(self.architectures),
            "model_type": "llama",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling.to_dict() if self.rope_scaling else None,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
            "mlp_bias": False,
        }
        if self.eos_token_id:
            d["eos_token_id"] = list(self.eos_token_id) if len(self.eos_token_id) > 1 else self.eos_token_id[0]
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.torch_dtype:
            d["torch_dtype"] = self.torch_dtype
        return d

    def num_parameters(self) -> int:
        h, i, v = self.hidden_size, self.intermediate_size, self.vocab_size
        q, kv = self.num_attention_heads * self.head_dim, self.num_key_value_heads * self.head_dim
        per_layer = (q + 2 * kv) * h + h * q + 3 * i * h + 2 * h
        return self.num_hidden_layers * per_layer + v * h * (1 if self.tie_word_embeddings else 2) + h


__all__ = ["ConfigError", "RopeScaling", "LlamaConfig", "asdict"]
