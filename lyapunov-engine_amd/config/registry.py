"""Registries: from a name to the class or function that builds the thing.

``ARCHITECTURES`` maps the string in config.json's ``architectures`` list to an
architecture (a typed configuration class plus a function that turns such a
configuration into a ``ModelSpec``).  ``MIXERS``, ``FEED_FORWARDS``, ``NORMS``,
``POSITION_ENCODINGS``, ``BLOCKS``, ``EMBEDDINGS`` and ``HEADS`` map a
``PartSpec.kind`` to a part class.
Code outside this package (a test, a plug-in) adds an entry with
``@REGISTRY.register("name")`` and needs no change to the package's files.

The reference has no registry: ``from_pretrained_llama`` names its one class
(python/lyapunov_engine/models/weight_loader.py:174-183).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable


class Registry:
    def __init__(self, what: str):
        self.what = what
        self._entries: dict[str, Any] = {}

    def register(self, name: str, obj: Any = None, *, replace: bool = False):
        def put(o):
            if name in self._entries and not replace:
                raise KeyError(f"{self.what} {name!r} is already registered")
            self._entries[name] = o
            return o

        return put if obj is None else put(obj)

    def unregister(self, name: str) -> None:
        self._entries.pop(name, None)

    def get(self, name: str) -> Any:
        try:
            return self._entries[name]
        except KeyError:
            raise KeyError(f"unknown {self.what} {name!r}; known: {sorted(self._entries)}") from None

    def __contains__(self, name: str) -> bool:
        return name in self._entries

    def names(self) -> list[str]:
        return sorted(self._entries)

    def build(self, spec, **extra):
        """Construct the part a PartSpec names."""
        return self.get(spec.kind)(**spec.params, **extra)


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Any                       # has from_dict(dict) and to_dict()
    to_spec: Callable[[Any], Any]           # config -> ModelSpec


ARCHITECTURES = Registry("architecture")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block arrangement")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("output head")


def register_architecture(name: str, config_class: Any, to_spec: Callable[[Any], Any], *, replace: bool = False):
    return ARCHITECTURES.register(name, Architecture(name, config_class, to_spec), replace=replace)


def architecture_of(config_dict: dict) -> Architecture:
    """The architecture a config.json asks for: the first name of its
    ``architectures`` list that is registered."""
    names = config_dict.get("architectures")
    if not names:
        raise KeyError(f"config.json has no 'architectures' entry; known: {ARCHITECTURES.names()}")
    for n in names:
        if n in ARCHITECTURES:
            return ARCHITECTURES.get(n)
    raise KeyError(f"unknown architecture {list(names)}; known: {ARCHITECTURES.names()}")


def load_config(model_dir: str):
    """Read ``<model_dir>/config.json`` -> (architecture, its typed configuration)."""
    path = os.path.join(model_dir, "config.json")
    if not os.path.exists(path):
        raise FileNotFoundError(f"{model_dir} has no config.json")
    with open(path, "r", encoding="utf-8") as f:
        raw = json.load(f)
    # The end-of-sequence ids may stand in generation_config.json instead (the reference fixes
    # 128001 in its scheduler, csrc/include/engine/scheduler.hpp:16, and reads neither file for them).
    extra = os.path.join(model_dir, "generation_config.json")
    if raw.get("eos_token_id") is None and os.path.exists(extra):
        with open(extra, "r", encoding="utf-8") as f:
            eos = json.load(f).get("eos_token_id")
        if eos is not None:
            raw = dict(raw, eos_token_id=eos)
    arch = architecture_of(raw)
    return arch, arch.config_class.from_dict(raw)
