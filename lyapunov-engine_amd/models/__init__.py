"""Architectures.  Importing the package registers the built-in one."""
from . import llama  # noqa: F401
from .decoder import CacheGroupLayout, CacheLayout, DecoderModel, build_model

__all__ = ["CacheGroupLayout", "CacheLayout", "DecoderModel", "build_model"]
