"""Typed configuration, registry, and the structure a configuration turns into."""
import json

import pytest

from conftest import TINY_A, TINY_B
from lyapunov_engine_amd.config import (ARCHITECTURES, ConfigError, EngineConfig, LlamaConfig, MIXERS, architecture_of,
                                        load_config)
from lyapunov_engine_amd.models import build_model
from lyapunov_engine_amd.models.llama import llama_spec

LLAMA_1B = dict(
    architectures=["LlamaForCausalLM"], vocab_size=128256, hidden_size=2048, intermediate_size=8192,
    num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8, head_dim=64, max_position_embeddings=131072,
    rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True, eos_token_id=[128001, 128008, 128009],
    bos_token_id=128000, torch_dtype="bfloat16", hidden_act="silu", attention_bias=False, mlp_bias=False,
    rope_scaling=dict(factor=32.0, high_freq_factor=4.0, low_freq_factor=1.0, original_max_position_embeddings=8192,
                      rope_type="llama3"), model_type="llama", transformers_version="4.45.0")


def test_every_size_comes_from_the_file():
    cfg = LlamaConfig.from_dict(LLAMA_1B)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.intermediate_size, cfg.num_hidden_layers) == (128256, 2048, 8192, 16)
    assert (cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim) == (32, 8, 64)
    assert cfg.rope_scaling.rope_type == "llama3" and cfg.rope_scaling.factor == 32.0
    assert cfg.rope_scaling.original_max_position_embeddings == 8192
    assert cfg.tie_word_embeddings and cfg.eos_token_id == (128001, 128008, 128009) and cfg.bos_token_id == 128000
    assert cfg.num_parameters() == 1_235_814_400
    assert "transformers_version" in cfg.extra  # unknown keys are kept aside, not an error
    # a missing size is an error, not a silent default of some model
    for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                "max_position_embeddings", "rms_norm_eps"):
        d = dict(LLAMA_1B)
        del d[key]
        with pytest.raises(ConfigError, match=key):
            LlamaConfig.from_dict(d)


def test_conventional_fallbacks():
    d = dict(TINY_A)
    del d["head_dim"], d["num_key_value_heads"], d["tie_word_embeddings"], d["rope_scaling"], d["rope_theta"]
    cfg = LlamaConfig.from_dict(d)
    assert cfg.rope_theta == 10000.0        # the file format's convention, not some model's value (weight_loader.py:37 says 500000)
    assert cfg.head_dim == 64 // 4          # hidden_size // heads (reference: weight_loader.py:30-34)
    assert cfg.num_key_value_heads == 4     # as many as query heads
    assert cfg.tie_word_embeddings is False and cfg.rope_scaling is None
    assert LlamaConfig.from_dict(dict(TINY_A, eos_token_id=7)).eos_token_id == (7,)
    assert LlamaConfig.from_dict(dict(TINY_A, rope_scaling={"rope_type": "default"})).rope_scaling is None


@pytest.mark.parametrize("bad,match", [
    (dict(num_key_value_heads=3), "do not split"),
    (dict(head_dim=15), "even"),
    (dict(attention_bias=True), "bias"),
    (dict(hidden_act="gelu"), "hidden_act"),
    (dict(rope_scaling={"rope_type": "yarn", "factor": 2.0}), "yarn"),
    (dict(rope_scaling={"rope_type": "llama3", "factor": 8.0}), "lacks"),
    (dict(vocab_size=0), "positive"),
    (dict(eos_token_id=999), "outside"),
    (dict(rms_norm_eps=0.0), "rms_norm_eps"),
])
def test_what_is_not_implemented_is_refused(bad, match):
    with pytest.raises(ConfigError, match=match):
        LlamaConfig.from_dict(dict(TINY_A, **bad))


@pytest.mark.parametrize("head_dim", [24, 272])
def test_a_head_size_the_kernels_do_not_take_is_refused_when_the_model_is_built(head_dim):
    """The configuration is a valid Llama configuration; it is the attention
    kernels that exist for multiples of 16 up to 256 only, and the part says so."""
    from lyapunov_engine_amd.models import build_model
    from lyapunov_engine_amd.models.llama import llama_spec

    cfg = LlamaConfig.from_dict(dict(TINY_A, head_dim=head_dim))
    with pytest.raises(ValueError, match="multiples of 16"):
        build_model(llama_spec(cfg))


def test_round_trip_through_json(tmp_path):
    for raw in (TINY_A, TINY_B, LLAMA_1B):
        cfg = LlamaConfig.from_dict(raw)
        (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
        arch, again = load_config(str(tmp_path))
        assert arch.name == "LlamaForCausalLM" and again == cfg


def test_registry_picks_the_model_by_name():
    assert architecture_of({"architectures": ["LlamaForCausalLM"]}) is ARCHITECTURES.get("LlamaForCausalLM")
    assert architecture_of({"architectures": ["Nope", "LlamaForCausalLM"]}).name == "LlamaForCausalLM"
    with pytest.raises(KeyError, match="LlamaForCausalLM"):   # the error lists what is known
        architecture_of({"architectures": ["MixtralForCausalLM"]})
    with pytest.raises(KeyError, match="architectures"):
        architecture_of({})
    assert "paged_attention" in MIXERS
    with pytest.raises(KeyError, match="already registered"):
        MIXERS.register("paged_attention", object)


def test_end_of_sequence_ids_may_stand_in_generation_config(tmp_path):
    import json

    from lyapunov_engine_amd.config.registry import load_config

    d = dict(TINY_A)
    d.pop("eos_token_id", None)
    (tmp_path / "config.json").write_text(json.dumps(d))
    assert load_config(str(tmp_path))[1].eos_token_id == ()
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [5, 9], "temperature": 0.6}))
    assert load_config(str(tmp_path))[1].eos_token_id == (5, 9)
    (tmp_path / "config.json").write_text(json.dumps(dict(d, eos_token_id=7)))   # config.json wins when it names them
    assert load_config(str(tmp_path))[1].eos_token_id == (7,)
    with pytest.raises(FileNotFoundError, match="config.json"):
        load_config(str(tmp_path / "nowhere"))


def test_the_two_tiny_configurations_differ_in_everything():
    a, b = LlamaConfig.from_dict(TINY_A), LlamaConfig.from_dict(TINY_B)
    for f in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
              "num_key_value_heads", "head_dim", "max_position_embeddings", "rms_norm_eps", "rope_theta",
              "rope_scaling", "tie_word_embeddings"):
        assert getattr(a, f) != getattr(b, f), f
    assert a.num_attention_heads // a.num_key_value_heads != b.num_attention_heads // b.num_key_value_heads
    assert a.intermediate_size % 8 and b.vocab_size % 2  # widths that are no power of two


def test_model_structure_follows_the_configuration():
    for raw in (TINY_A, TINY_B):
        cfg = LlamaConfig.from_dict(raw)
        model = build_model(llama_spec(cfg))
        names = model.expected_tensors()
        H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
        q, kv = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
        assert names["model.embed_tokens.weight"][0] == (V, H)
        assert ("lm_head.weight" in names) == (not cfg.tie_word_embeddings)
        last = cfg.num_hidden_layers - 1
        assert names[f"model.layers.{last}.self_attn.q_proj.weight"][0] == (q, H)
        assert names[f"model.layers.{last}.self_attn.k_proj.weight"][0] == (kv, H)
        assert names[f"model.layers.0.self_attn.o_proj.weight"][0] == (H, q)
        assert names[f"model.layers.0.mlp.gate_proj.weight"][0] == (I, H)
        assert names[f"model.layers.0.mlp.down_proj.weight"][0] == (H, I)
        assert names["model.norm.weight"] == ((H,), "ones")
        assert len(names) == 9 * cfg.num_hidden_layers + 2 + (0 if cfg.tie_word_embeddings else 1)
        layout = model.cache_layout()
        assert len(layout.groups) == 1 and layout.groups[0].buffers == tuple(range(cfg.num_hidden_layers))
        from lyapunov_engine_amd.parts import SLOT
        k, v = layout.groups[0].spec.tensors      # the layout is the mixer's: keys [heads][slot][hd], values [heads][hd][slot]
        assert (k.name, k.shape) == ("k", (cfg.num_key_value_heads, SLOT, cfg.head_dim)) and not layout.states
        assert (v.name, v.shape) == ("v", (cfg.num_key_value_heads, cfg.head_dim, SLOT))
        assert k.page_shape(16) == (cfg.num_key_value_heads, 16, cfg.head_dim)
        assert sum(1 for _ in model.named_parts()) > 0
        total = sum(int(__import__("math").prod(s)) for s, _ in names.values())
        assert total == cfg.num_parameters()


def test_engine_config_names_follow_the_reference():
    c = EngineConfig()
    assert (c.num_blocks, c.block_size, c.max_num_seqs, c.max_num_batched_tokens) == (1024, 16, 64, 2048)
    assert EngineConfig(num_gpu_blocks=77).num_blocks == 77     # the alias (llm_engine.py:33)
    import torch
    assert EngineConfig(dtype="float32").dtype == torch.float32 and EngineConfig(dtype="bf16").dtype == torch.bfloat16
    with pytest.raises(ValueError):
        EngineConfig(dtype="float16")
    with pytest.raises(ValueError):
        EngineConfig(block_size=0)


def test_layers_with_equal_position_parameters_share_one_table():
    """A model of the 1B shape's depth with 131,072 positions holds one table of cosines and sines
    (131,072 x 64 floats = 32 MiB), not one per layer; an engine that will never reach beyond 4,096
    positions builds 4,096 rows."""
    import torch

    from lyapunov_engine_amd.models import build_model
    from lyapunov_engine_amd.models.llama import llama_spec

    raw = dict(architectures=["LlamaForCausalLM"], vocab_size=64, hidden_size=128, intermediate_size=64,
               num_hidden_layers=16, num_attention_heads=2, num_key_value_heads=1, head_dim=64,
               max_position_embeddings=131072, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True,
               rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=8192))
    model = build_model(llama_spec(LlamaConfig.from_dict(raw)))
    model.materialize("cpu", torch.float32)
    tables = [layer.mixer.position.table for layer in model.layers]
    assert len({t.data_ptr() for t in tables}) == 1 and all(t is tables[0] for t in tables)
    assert tables[0].shape == (131072, 64) and tables[0].numel() * 4 == 32 << 20
    assert model.max_positions == 131072

    small = build_model(llama_spec(LlamaConfig.from_dict(raw)))
    small.materialize("cpu", torch.float32, max_positions=4096)
    assert small.layers[0].mixer.position.table.shape == (4096, 64) and small.max_positions == 4096
    torch.testing.assert_close(small.layers[0].mixer.position.table, tables[0][:4096], rtol=0, atol=0)
    # other parameters, another table
    other = build_model(llama_spec(LlamaConfig.from_dict(dict(raw, rope_theta=10000.0, max_position_embeddings=4096))))
    other.materialize("cpu", torch.float32)
    assert other.layers[0].mixer.position.table.data_ptr() != small.layers[0].mixer.position.table.data_ptr()


def test_embedding_and_head_are_parts_an_architecture_may_replace():
    """The model's two ends come from registries like every other part: the built-in kinds bind the
    usual two tensors (one when tied, and then the head uses the embedding's matrix itself); kinds
    registered from outside bring their own tensors and constants, a head that cannot share the
    embedding's matrix says so, and an unknown kind names the known ones."""
    import dataclasses

    import torch

    from lyapunov_engine_amd.config import EMBEDDINGS, HEADS, PartSpec
    from lyapunov_engine_amd.parts import Embedding, Head, WeightSource, WeightSpec

    tied = build_model(llama_spec(LlamaConfig.from_dict(TINY_A)))
    assert type(tied.embedding).__name__ == "TokenEmbedding" and type(tied.head).__name__ == "LinearHead"
    assert "lm_head.weight" not in tied.expected_tensors() and tied.ignorable("lm_head.weight")
    tied.embedding.weight = torch.zeros(3, 2)
    tied.materialize("cpu", torch.float32)
    assert tied.lm_head is tied.embed and tied.head.weight is tied.embedding.weight     # one matrix, two uses
    untied = build_model(llama_spec(LlamaConfig.from_dict(TINY_B)))
    assert "lm_head.weight" in untied.expected_tensors() and not untied.ignorable("lm_head.weight")

    class Scaled(Embedding):
        def __init__(self, vocab_size, hidden_size, scale):
            self.sizes, self.scale, self.weight = (vocab_size, hidden_size), scale, None

        def weight_specs(self):
            return [WeightSpec("weight", (WeightSource("weight", self.sizes),)),
                    WeightSpec("offset", (WeightSource("offset", (self.sizes[1],)),))]

    class Biased(Head):
        def __init__(self, vocab_size, hidden_size):
            self.vocab_size, self.shared = vocab_size, None

        def tie(self, embedding):
            self.shared = embedding

        def weight_specs(self):
            return [WeightSpec("bias", (WeightSource("bias", (self.vocab_size,)),))]

    class Alone(Head):          # keeps the default tie(): it cannot share
        def __init__(self, vocab_size, hidden_size):
            pass

    EMBEDDINGS.register("test_scaled", Scaled)
    HEADS.register("test_biased", Biased)
    HEADS.register("test_alone", Alone)
    try:
        spec = dataclasses.replace(llama_spec(LlamaConfig.from_dict(TINY_A)), embedding=PartSpec("test_scaled", {"scale": 3.0}),
                                   head=PartSpec("test_biased"), embed_prefix="tok.", head_prefix="out.")
        model = build_model(spec)
        names = model.expected_tensors()
        assert names["tok.weight"][0] == (TINY_A["vocab_size"], TINY_A["hidden_size"]) and names["tok.offset"][0] == (TINY_A["hidden_size"],)
        assert names["out.bias"][0] == (TINY_A["vocab_size"],) and "lm_head.weight" not in names and "model.embed_tokens.weight" not in names
        assert model.embedding.scale == 3.0 and model.head.shared is model.embedding
        assert model.ignorable("out.weight") and not model.ignorable("lm_head.weight")   # tied: the head's prefix
        with pytest.raises(NotImplementedError, match="cannot share"):
            build_model(dataclasses.replace(spec, head=PartSpec("test_alone")))
        with pytest.raises(KeyError, match="unknown output head 'nope'.*linear"):
            build_model(dataclasses.replace(spec, head=PartSpec("nope")))
    finally:
        EMBEDDINGS.unregister("test_scaled")
        HEADS.unregister("test_biased")
        HEADS.unregister("test_alone")


def test_one_switch_decides_what_is_said(capsys, monkeypatch):
    from lyapunov_engine_amd.utils import log

    before = log.level()
    try:
        log.set_level("quiet")
        log.info("progress"), log.debug("counters"), log.warn("switched off")
        assert capsys.readouterr().err == "[lyapunov-amd] switched off\n"
        log.set_level("info")
        log.info("progress"), log.debug("counters")
        assert capsys.readouterr().err == "[lyapunov-amd] progress\n"
        log.set_level("debug")
        log.debug("counters")
        assert "counters" in capsys.readouterr().err
        with pytest.raises(ValueError, match="one of"):
            log.set_level("loud")
    finally:
        log.set_level(before)
