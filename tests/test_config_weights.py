"""Configuration, registry and weight loading (no GPU)."""
import json
import os

import pytest
import torch

from util import TINY_A, TINY_B

from tiny_llm_amd.config import (ConfigError, EngineConfig, LlamaConfig, UnknownArchitecture, known_architectures,
                                 resolve)
from tiny_llm_amd.models.decoder import Decoder
from tiny_llm_amd.weights import (SafetensorsError, SafetensorsFile, WeightLoadError, check_against, save_file,
                                  write_random_model)
from tiny_llm_amd.weights.loader import load_weights, random_tensor, target_dtype
from tiny_llm_amd.parts.base import WeightSpec


def test_reference_config_file_parses_to_tinyllama_sizes():
    # the reference's own fixture (tests/datas/llama_config.json), as tests/parser/test_llama_parser.cpp:12-20 reads it
    path = "/root/reference/tests/datas/llama_config.json"
    if not os.path.exists(path):
        pytest.skip("reference checkout not mounted")
    cfg = LlamaConfig.from_json(path)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads) == (22, 2048, 32, 4)
    assert (cfg.head_dim, cfg.intermediate_size, cfg.vocab_size, cfg.max_position_embeddings) == (64, 5632, 32000, 2048)
    assert cfg.rope_theta == 10000.0 and cfg.rms_norm_eps == 1e-5 and not cfg.tie_word_embeddings
    assert cfg.eos_token_id == 2


def test_defaults_and_head_dim_key():
    d = {"architectures": ["LlamaForCausalLM"], "vocab_size": 10, "hidden_size": 32, "intermediate_size": 48,
         "num_hidden_layers": 1, "num_attention_heads": 4}
    cfg = LlamaConfig.from_dict(d)
    assert cfg.num_key_value_heads == 4 and cfg.head_dim == 8 and cfg.rope_theta == 10000.0
    assert cfg.rms_norm_eps == 1e-6 and not cfg.tie_word_embeddings and cfg.hidden_act == "silu"
    cfg = LlamaConfig.from_dict(dict(d, head_dim=16, num_key_value_heads=2))
    assert cfg.head_dim == 16 and cfg.num_key_value_heads == 2


@pytest.mark.parametrize("patch,word", [
    ({"attention_bias": True}, "bias"), ({"rope_scaling": {"type": "linear"}}, "rope_scaling"),
    ({"hidden_act": "gelu"}, "hidden_act"), ({"num_key_value_heads": 3}, "multiple"),
    ({"hidden_size": 65}, "head_dim"), ({"vocab_size": None}, "vocab_size"), ({"rms_norm_eps": 0}, "rms_norm_eps"),
])
def test_refusals(patch, word):
    # the reference refuses biases, rope scaling and other activations (llama_parser.cpp:165-169)
    d = dict(TINY_A)
    d.update(patch)
    with pytest.raises(ConfigError) as e:
        LlamaConfig.from_dict(d)
    assert word in str(e.value)


def test_registry_chooses_by_architecture_name():
    assert "LlamaForCausalLM" in known_architectures()
    cfg, spec = resolve(TINY_B)
    assert spec.architecture == "LlamaForCausalLM" and len(spec.layers) == 3 and len(spec.plan) == 3
    assert spec.layers[1].mixer.kind == "attention" and spec.layers[1].ffn.kind == "swiglu"
    assert spec.layers[0].mixer.params["position"]["theta"] == 500000.0
    assert spec.lm_head.params["tied"] is True
    with pytest.raises(UnknownArchitecture) as e:
        resolve(dict(TINY_A, architectures=["MambaForCausalLM"]))
    assert "LlamaForCausalLM" in str(e.value)


def test_no_size_stands_in_code():
    """Every size of the built parts comes from the configuration."""
    odd = dict(TINY_A, hidden_size=80, num_attention_heads=5, num_key_value_heads=5, head_dim=16,
               intermediate_size=72, vocab_size=99, num_hidden_layers=4)
    _, spec = resolve(odd)
    dec = Decoder(spec, "float32", "cpu")
    shapes = {s.name: s.shape for s in dec.weight_specs()}
    assert shapes["model.embed_tokens.weight"] == (99, 80)
    assert shapes["model.layers.3.self_attn.q_proj.weight"] == (80, 80)
    assert shapes["model.layers.3.self_attn.k_proj.weight"] == (80, 80)
    assert shapes["model.layers.0.mlp.down_proj.weight"] == (80, 72)
    assert shapes["lm_head.weight"] == (99, 80)
    assert len(shapes) == 3 + 4 * 9


def test_engine_config_checks():
    assert EngineConfig(dtype="bf16").dtype == "bfloat16" and EngineConfig(dtype="fp32").dtype == "float32"
    with pytest.raises(ValueError):
        EngineConfig(dtype="float16")
    with pytest.raises(ValueError):
        EngineConfig(kv_block_size=0)


# ------------------------------------------------------------------ safetensors
def test_safetensors_reader_vectors(tmp_path):
    # (ref) tests/weight_managers/test_safetensors.cpp:12-56: embedding [2,3] = 0..5, attention [2,2] = 10..13
    path = str(tmp_path / "t.safetensors")
    save_file({"embedding": torch.arange(6, dtype=torch.float32).reshape(2, 3),
               "attention": torch.arange(10, 14, dtype=torch.float32).reshape(2, 2)}, path)
    f = SafetensorsFile(path)
    assert sorted(f.names()) == ["attention", "embedding"]
    assert f.info("embedding") == (torch.float32, (2, 3))
    assert f.get("embedding").tolist() == [[0, 1, 2], [3, 4, 5]]
    assert f.get("attention").tolist() == [[10, 11], [12, 13]]
    with pytest.raises(SafetensorsError):
        f.get("missing")
    # the library's reader agrees with our writer, and ours with the library's writer
    from safetensors.torch import load_file, save_file as lib_save
    assert load_file(path)["attention"].tolist() == [[10, 11], [12, 13]]
    lib_save({"x": torch.tensor([1.5, -2.0], dtype=torch.bfloat16), "i": torch.tensor([[7]], dtype=torch.int32)},
             str(tmp_path / "lib.safetensors"))
    g = SafetensorsFile(str(tmp_path / "lib.safetensors"))
    assert g.get("x").dtype == torch.bfloat16 and g.get("x").tolist() == [1.5, -2.0] and g.get("i").item() == 7


def test_safetensors_rejects_damaged_files(tmp_path):
    p = tmp_path / "short.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(SafetensorsError):
        SafetensorsFile(str(p))
    p.write_bytes((10 ** 9).to_bytes(8, "little") + b"{}")
    with pytest.raises(SafetensorsError):
        SafetensorsFile(str(p))
    with pytest.raises(SafetensorsError):
        SafetensorsFile(str(tmp_path / "absent.safetensors"))


# ---------------------------------------------------------------------- loading
def _specs(cfg):
    _, spec = resolve(cfg)
    return Decoder(spec, "float32", "cpu")


def test_random_model_folder_round_trip(tmp_path):
    folder = write_random_model(str(tmp_path), TINY_A, seed=5)
    assert json.load(open(os.path.join(folder, "config.json")))["hidden_size"] == 64
    dec = _specs(TINY_A)
    load_weights(dec, folder)       # device "cpu": binding needs no kernel
    assert dec.layers[0].mixer.w_qkv.shape == ((4 + 2 * 2) * 16, 64)
    assert dec.layers[1].ffn.w_gate_up.shape == (2 * 176, 64)
    assert dec.lm_head.weight.shape == (251, 64)
    # the same (seed, name) gives the same tensor whatever else is generated, another seed another one
    again = write_random_model(str(tmp_path / "again"), TINY_A, seed=5)
    other = write_random_model(str(tmp_path / "other"), TINY_A, seed=6)
    a = SafetensorsFile(os.path.join(folder, "model.safetensors")).get("model.layers.1.mlp.up_proj.weight")
    b = SafetensorsFile(os.path.join(again, "model.safetensors")).get("model.layers.1.mlp.up_proj.weight")
    c = SafetensorsFile(os.path.join(other, "model.safetensors")).get("model.layers.1.mlp.up_proj.weight")
    assert torch.equal(a, b) and not torch.equal(a, c)
    assert abs(float(a.std()) - 0.02) < 0.002
    spec = WeightSpec("model.layers.1.mlp.up_proj.weight", (176, 64))
    assert torch.equal(random_tensor(spec, 5, 0.02, 0.0), a)


def test_tied_head_is_not_stored_and_shares_the_table(tmp_path):
    folder = write_random_model(str(tmp_path), TINY_B, seed=1, norm_std=0.1)
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    assert "lm_head.weight" not in f
    dec = _specs(TINY_B)
    load_weights(dec, folder)
    assert dec.lm_head.weight.data_ptr() == dec.embedding.weight.data_ptr()
    norm = f.get("model.layers.2.input_layernorm.weight")
    assert 0.03 < float(norm.std()) < 0.3 and abs(float(norm.mean()) - 1) < 0.1


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = write_random_model(str(tmp_path), TINY_A, seed=5)
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.get(n).clone() for n in f.names()}
    del f
    del tensors["model.layers.0.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.1.self_attn.o_proj.weight"] = torch.zeros(64, 32)
    tensors["model.layers.7.mlp.up_proj.weight"] = torch.zeros(2, 2)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)      # known and ignorable
    save_file(tensors, path)
    with pytest.raises(WeightLoadError) as e:
        load_weights(_specs(TINY_A), folder)
    err = e.value
    assert sorted(err.missing) == ["model.layers.0.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.mlp.up_proj.weight"]
    assert [(n, exp, got) for n, exp, got in err.wrong_shape] == [
        ("model.layers.1.self_attn.o_proj.weight", (64, 64), (64, 32))]
    text = str(err)
    for word in ("missing", "unexpected", "wrong shapes", "model.norm.weight", "[64, 32]"):
        assert word in text


def test_untied_model_needs_its_head(tmp_path):
    folder = write_random_model(str(tmp_path), TINY_B, seed=1)
    cfg = dict(TINY_B, tie_word_embeddings=False)
    with pytest.raises(WeightLoadError) as e:
        load_weights(_specs(cfg), folder)
    assert e.value.missing == ["lm_head.weight"]


def test_element_types():
    m = WeightSpec("w", (2, 2), role="matrix")
    v = WeightSpec("n", (2,), role="vector")
    t = WeightSpec("t", (2,), role="table")
    bf, f32 = torch.bfloat16, torch.float32
    assert target_dtype(m, f32, bf) == bf and target_dtype(m, bf, f32) == f32
    assert target_dtype(v, f32, bf) == f32            # stored in 32 bits: stays so
    assert target_dtype(v, bf, bf) == bf and target_dtype(v, bf, f32) == f32
    assert target_dtype(t, torch.int64, bf) == torch.int32


def test_bf16_folder_loads_into_both_engine_types(tmp_path):
    folder = write_random_model(str(tmp_path), TINY_A, seed=2, dtype="bfloat16")
    assert json.load(open(os.path.join(folder, "config.json")))["torch_dtype"] == "bfloat16"
    _, spec = resolve(TINY_A)
    for dt in ("float32", "bfloat16"):
        dec = Decoder(spec, dt, "cpu")
        load_weights(dec, folder)
        assert dec.layers[0].mixer.w_o.dtype == dec.dtype
        assert dec.final_norm.weight.dtype == dec.dtype
