from .engine_config import EngineConfig, parse_dtype
from .model_config import ConfigError, LlamaConfig, RopeScaling
from .registry import (ARCHITECTURES, BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS,
                       Architecture, Registry, architecture_of, load_config, register_architecture)
from .specs import HF_LAYER_NAMES, HF_PREFIXES, LayerCall, LayerSpec, ModelSpec, PartSpec, default_schedule

__all__ = [
    "EngineConfig", "parse_dtype", "ConfigError", "LlamaConfig", "RopeScaling", "ARCHITECTURES", "BLOCKS",
    "EMBEDDINGS", "HEADS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Architecture", "Registry", "architecture_of",
    "load_config", "register_architecture", "LayerCall", "LayerSpec", "ModelSpec", "PartSpec", "default_schedule",
    "HF_LAYER_NAMES", "HF_PREFIXES",
]
