"""Safetensors reader and writer, binding by name, the one error that lists
what is wrong, precision rules, and the random-weights mode."""
import json
import os
import struct

import pytest
import torch

from conftest import TINY_A, TINY_B
from lyapunov_engine_amd.config import LlamaConfig
from lyapunov_engine_amd.models import build_model
from lyapunov_engine_amd.models.llama import llama_spec
from lyapunov_engine_amd.weights import (DictSource, SafetensorsError, SafetensorsFile, WeightError, load_model,
                                         load_weights, random_tensors, write_random_model, write_safetensors)


def test_writer_and_reader_agree_with_the_safetensors_library(tmp_path):
    from safetensors.torch import load_file, save_file

    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int64),
               "d": torch.randn(2, 2, 2).half(), "e": torch.zeros(0, 4)}
    ours, theirs = str(tmp_path / "ours.safetensors"), str(tmp_path / "theirs.safetensors")
    write_safetensors(ours, tensors, metadata={"format": "pt"})
    save_file(tensors, theirs)
    back = load_file(ours)                      # the library reads what we wrote
    f = SafetensorsFile(theirs)                 # we read what the library wrote
    assert sorted(f.names()) == sorted(tensors)
    for k, v in tensors.items():
        assert torch.equal(back[k], v) and torch.equal(f.tensor(k), v) and f.tensor(k).dtype == v.dtype
    assert SafetensorsFile(ours).metadata == {"format": "pt"}


def test_broken_files_are_refused(tmp_path):
    p = tmp_path / "x.safetensors"
    p.write_bytes(b"abc")
    with pytest.raises(SafetensorsError, match="too short"):
        SafetensorsFile(str(p))
    p.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(str(p))
    hdr = json.dumps({"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="needs 16"):
        SafetensorsFile(str(p))
    hdr = json.dumps({"t": {"dtype": "F8_E4M3", "shape": [4], "data_offsets": [0, 4]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 4)
    with pytest.raises(SafetensorsError, match="unknown dtype"):
        SafetensorsFile(str(p))
    empty = tmp_path / "empty"
    empty.mkdir()
    (empty / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(FileNotFoundError, match="no .safetensors"):   # weight_loader.py:50-53
        load_model(str(empty), torch.float32, "cpu")
    with pytest.raises(FileNotFoundError, match="config.json"):
        load_model(str(tmp_path / "nowhere"), torch.float32, "cpu")


def make(cfg_dict):
    cfg = LlamaConfig.from_dict(cfg_dict)
    return cfg, build_model(llama_spec(cfg))


def test_random_weights_depend_on_seed_and_name_only():
    _, model = make(TINY_A)
    a = dict(random_tensors(model, 0, torch.float32))
    b = dict(random_tensors(model, 0, torch.float32))
    c = dict(random_tensors(model, 1, torch.float32))
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    assert a["model.layers.0.input_layernorm.weight"].eq(1).all()             # norm weights are ones
    assert abs(float(a["model.embed_tokens.weight"].std()) - 0.02) < 2e-3     # matrices ~ N(0, 0.02)
    noisy = dict(random_tensors(model, 0, torch.float32, norm_init_std=0.1))
    assert 0.05 < float(noisy["model.norm.weight"].std()) < 0.2
    # a deeper model of the same seed has the same first layers: values do not depend on generation order
    _, deeper = make(dict(TINY_A, num_hidden_layers=3))
    d = dict(random_tensors(deeper, 0, torch.float32))
    assert all(torch.equal(a[k], d[k]) for k in a)


def test_folder_round_trip_and_fusing(tmp_path):
    for raw, dtype in ((TINY_A, "float32"), (TINY_B, "bfloat16")):
        d = str(tmp_path / f"m{raw['hidden_size']}")
        write_random_model(dict(raw), d, seed=3, dtype=dtype, norm_init_std=0.1)
        assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
        assert json.load(open(os.path.join(d, "config.json")))["torch_dtype"] == dtype
        model, cfg = load_model(d, torch.float32, "cpu")
        f = SafetensorsFile(os.path.join(d, "model.safetensors"))
        p = "model.layers.1."
        att, ffn = model.layers[1].mixer, model.layers[1].ffn
        want_qkv = torch.cat([f.tensor(p + f"self_attn.{n}_proj.weight").float() for n in "qkv"], 0)
        assert torch.equal(att.qkv_proj, want_qkv)                 # q, k, v rows in this order
        gate, up = f.tensor(p + "mlp.gate_proj.weight").float(), f.tensor(p + "mlp.up_proj.weight").float()
        assert ffn.gate_up_proj.shape == (2 * cfg.intermediate_size, cfg.hidden_size)
        if ffn.interleave:                                          # tiles of 16 rows: eight gates, their eight ups
            tiles = ffn.gate_up_proj.view(-1, 2, 8, cfg.hidden_size)
            assert torch.equal(tiles[:, 0].reshape(gate.shape), gate) and torch.equal(tiles[:, 1].reshape(up.shape), up)
        else:                                                       # gate rows first (weight_loader.py:155-163)
            assert torch.equal(ffn.gate_up_proj, torch.cat([gate, up], 0))
        assert bool(ffn.interleave) == (cfg.intermediate_size % 8 == 0)
        assert torch.equal(model.layers[1].norm2.weight, f.tensor(p + "post_attention_layernorm.weight").float())
        if cfg.tie_word_embeddings:
            assert model.lm_head is model.embed                     # one matrix, two uses
        else:
            assert torch.equal(model.lm_head, f.tensor("lm_head.weight").float())


def test_precision_rules(tmp_path):
    cfg, model = make(TINY_A)
    t = dict(random_tensors(model, 0, torch.bfloat16))
    t["model.norm.weight"] = t["model.norm.weight"].float()                       # stored in 32-bit
    t["model.layers.0.self_attn.k_proj.weight"] = t["model.layers.0.self_attn.k_proj.weight"].float()
    t["model.layers.1.mlp.down_proj.weight"] = t["model.layers.1.mlp.down_proj.weight"].half()
    load_weights(model, DictSource(t), torch.bfloat16, "cpu")
    assert model.embed.dtype == torch.bfloat16                                     # kept in bfloat16
    assert model.final_norm.weight.dtype == torch.float32                          # a 32-bit tensor stays so
    assert model.layers[0].mixer.qkv_proj.dtype == torch.float32                   # a fused matrix with a 32-bit piece
    assert model.layers[1].mixer.qkv_proj.dtype == torch.bfloat16
    assert model.layers[1].ffn.down_proj.dtype == torch.bfloat16                   # float16 becomes bfloat16
    _, model32 = make(TINY_A)
    load_weights(model32, DictSource(t), torch.float32, "cpu")
    assert {w.dtype for w in (model32.embed, model32.layers[1].ffn.down_proj, model32.final_norm.weight)} == {torch.float32}


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    cfg, model = make(TINY_B)
    t = dict(random_tensors(model, 0, torch.float32))
    del t["model.layers.2.mlp.up_proj.weight"], t["lm_head.weight"]
    t["model.layers.0.self_attn.extra_bias"] = torch.zeros(16)
    t["model.layers.1.self_attn.q_proj.weight"] = torch.zeros(96, 95)
    t["model.norm.weight"] = torch.zeros(97)
    with pytest.raises(WeightError) as e:
        load_weights(model, DictSource(t), torch.float32, "cpu")
    msg = str(e.value)
    assert "missing (2)" in msg and "model.layers.2.mlp.up_proj.weight" in msg and "lm_head.weight" in msg
    assert "unexpected (1)" in msg and "self_attn.extra_bias" in msg
    assert "wrong shape (2)" in msg and "q_proj.weight is [96, 95], expected [96, 96]" in msg and "model.norm.weight" in msg


def test_a_tied_model_ignores_a_separate_head(capsys):
    cfg, model = make(TINY_A)
    t = dict(random_tensors(model, 0, torch.float32))
    t["lm_head.weight"] = torch.zeros(256, 64)
    load_weights(model, DictSource(t), torch.float32, "cpu")
    assert model.lm_head is model.embed and "lm_head.weight" in capsys.readouterr().err


def test_buffers_the_architecture_declares_ignorable_do_not_stop_loading(capsys):
    """Older exports store every layer's rotary frequencies; the model computes its own."""
    cfg, model = make(TINY_B)
    t = dict(random_tensors(model, 0, torch.float32))
    for i in range(cfg.num_hidden_layers):
        t[f"model.layers.{i}.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    load_weights(model, DictSource(t), torch.float32, "cpu")
    assert "rotary_emb.inv_freq" in capsys.readouterr().err
    t["model.layers.0.self_attn.rotary_emb.cos_cached"] = torch.zeros(4)     # not declared: still an error
    with pytest.raises(WeightError, match="unexpected"):
        load_weights(model, DictSource(t), torch.float32, "cpu")
