"""The Llama architecture as a ModelSpec: which parts, with which sizes, under
which tensor names.

Layer by layer this is the reference's LlamaDecoderLayer
(python/lyapunov_engine/models/llama.py:125-165): RMSNorm, grouped-query
attention with rotary encoding, RMSNorm, SiLU-gated feed-forward; the tensor
names are the ones its loader binds (models/weight_loader.py:91-169).  Not in the
reference: ``rope_scaling`` of type llama3 and ``tie_word_embeddings``.
"""
from __future__ import annotations

from ..config.model_config import LlamaConfig
from ..config.registry import register_architecture
from ..config.specs import HF_LAYER_NAMES, HF_PREFIXES, LayerSpec, ModelSpec, PartSpec, default_schedule


def llama_spec(cfg: LlamaConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    position = PartSpec("rope", {
        "dim": cfg.head_dim,
        "theta": cfg.rope_theta,
        "max_position": cfg.max_position_embeddings,
        "scaling": cfg.rope_scaling.to_dict() if cfg.rope_scaling else None,
    })
    mixer = PartSpec("paged_attention", {
        "hidden_size": cfg.hidden_size,
        "num_heads": cfg.num_attention_heads,
        "num_kv_heads": cfg.num_key_value_heads,
        "head_dim": cfg.head_dim,
        "position": position,
    })
    ffn = PartSpec("swiglu", {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size})
    layer = LayerSpec(block="prenorm", mixer=mixer, ffn=ffn, norm1=norm, norm2=norm, names=HF_LAYER_NAMES)
    return ModelSpec(
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        layers=tuple(layer for _ in range(cfg.num_hidden_layers)),
        schedule=default_schedule(cfg.num_hidden_layers),
        final_norm=norm,
        tie_word_embeddings=cfg.tie_word_embeddings,
        max_position=cfg.max_position_embeddings,
        eos_token_ids=tuple(cfg.eos_token_id),
        # older exports carry every layer's rotary frequencies as a buffer; they are computed here
        ignorable_tensors=("*.rotary_emb.inv_freq",),
        **HF_PREFIXES,   # model.embed_tokens., model.layers.{i}., model.norm., lm_head. (models/weight_loader.py:85-170)
    )


register_architecture("LlamaForCausalLM", LlamaConfig, llama_spec, replace=True)
