"""What an architecture hands to the model builder: a description, in plain
data, of which parts make up each layer and in which order the layers run.

Nothing in here knows Llama.  An architecture (``models/llama.py`` is the one in
this package) turns its own typed configuration into a ``ModelSpec``; the
builder (``models/decoder.py``) looks every part up by its kind in the
registries (the embedding and the output head too) and puts the model together.
Because the description is per layer, one model may use different mixers and
feed-forwards in different layers, and because the running order is a list of
its own, a layer may run twice or read the cache that another call of a layer
filled.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Mapping


@dataclass(frozen=True)
class PartSpec:
    """``kind`` names an entry of a registry; ``params`` are the constructor's
    keyword arguments (sizes and constants, never a model name)."""

    kind: str
    params: dict = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    block: str                      # arrangement of the parts, e.g. "prenorm"
    mixer: PartSpec
    ffn: PartSpec
    norm1: PartSpec                 # before the mixer
    norm2: PartSpec                 # before the feed-forward
    # Names of the four parts inside the layer's tensor-name prefix ("norm1", "mixer", "norm2",
    # "ffn" -> a piece of the tensor names); the architecture says what its files call them
    # (``HF_LAYER_NAMES`` is one convention an architecture may name).
    names: Mapping
    # Further parts for an arrangement that has more than these four (a norm
    # after each branch, a second feed-forward): name -> PartSpec; the block
    # kind decides which registry each comes from and what its tensors are
    # called.  "prenorm" takes none.
    extra: Mapping = field(default_factory=dict)

    def __post_init__(self):
        missing = [k for k in ("norm1", "mixer", "norm2", "ffn") if k not in self.names]
        if missing:
            raise ValueError(f"a layer's tensor names lack {missing}")
        for name, part in self.extra.items():
            if not isinstance(name, str) or not isinstance(part, PartSpec):
                raise ValueError(f"a layer's further parts are PartSpecs by name, not {name!r}: {part!r}")


@dataclass(frozen=True)
class LayerCall:
    """One entry of the running order.

    ``layer``   which LayerSpec (and so which weights) runs;
    ``cache``   which cache buffer its mixer uses; calls that name the same
                buffer share keys and values;
    ``writes``  false: the mixer only reads the buffer (another call filled it)
                and computes no keys and values of its own.
    """

    layer: int
    cache: int
    writes: bool = True


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    hidden_size: int
    layers: tuple                    # of LayerSpec
    schedule: tuple                  # of LayerCall
    final_norm: PartSpec
    tie_word_embeddings: bool       # the output head uses the embedding's matrix (Head.tie)
    max_position: int
    # The parts at the two ends, built with vocab_size= and hidden_size= beside
    # their own parameters: from token ids to the residual stream's first value,
    # and from normed rows to float logits.
    # Where the parts' tensors are found in the model's files: the architecture's own words
    # (``HF_PREFIXES`` is one convention an architecture may name).
    embed_prefix: str
    final_norm_prefix: str
    head_prefix: str
    layer_prefix: str                # with "{i}" for the layer's number
    embedding: PartSpec = PartSpec("lookup")
    head: PartSpec = PartSpec("linear")
    eos_token_ids: tuple = ()
    ignorable_tensors: tuple = ()    # shell-style patterns of tensor names a file may hold unused
    init_std: float = 0.02           # random-weights mode: normal(0, init_std) matrices
    norm_init_std: float = 0.0       # random-weights mode: norm weights 1 + normal(0, norm_init_std)


# The tensor names of decoder checkpoints in the Hugging Face convention, for architectures whose
# files follow it; nothing uses them unless an architecture's ``to_spec`` names them.
HF_LAYER_NAMES = {"norm1": "input_layernorm", "mixer": "self_attn", "norm2": "post_attention_layernorm", "ffn": "mlp"}
HF_PREFIXES = dict(embed_prefix="model.embed_tokens.", final_norm_prefix="model.norm.", head_prefix="lm_head.",
                   layer_prefix="model.layers.{i}.")


def default_schedule(n_layers: int) -> tuple:
    return tuple(LayerCall(i, i, True) for i in range(n_layers))


__all__ = ["PartSpec", "LayerSpec", "LayerCall", "ModelSpec", "default_schedule", "HF_LAYER_NAMES", "HF_PREFIXES"]
