"""Configuration, registry and weight loading (no GPU)."""
import json
import os

import pytest
import torch

from util import REFERENCE_DATA, TINY_A, TINY_B

from tiny_llm_amd.config import (ConfigError, EngineConfig, LlamaConfig, UnknownArchitecture, known_architectures,
                                 resolve)
from tiny_llm_amd.models.decoder import Decoder
from tiny_llm_amd.weights import (SafetensorsError, SafetensorsFile, WeightLoadError, check_against, save_file,
                                  write_random_model)
from tiny_llm_amd.weights.loader import load_weights, random_tensor, target_dtype
from tiny_llm_amd.parts.base import WeightSpec


def test_reference_config_file_parses_to_tinyllama_sizes():
    # the reference's own fixture (tests/datas/llama_config.json), as tests/parser/test_llama_parser.cpp:12-20 reads it
    path = os.path.join(REFERENCE_DATA, "llama_config.json")
    if not os.path.exists(path):
        pytest.skip("reference checkout not mounted")
    cfg = LlamaConfig.from_json(path)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads) == (22, 2048, 32, 4)
    assert (cfg.head_dim, cfg.intermediate_size, cfg.vocab_size, cfg.max_position_embeddings) == (64, 5632, 32000, 2048)
    assert cfg.rope_theta == 10000.0 and cfg.rms_norm_eps == 1e-5 and not cfg.tie_word_embeddings
    assert cfg.eos_token_id == 2 and cfg.eos_token_ids == (2,)


def test_every_end_of_sequence_id_is_kept():
    d = dict(TINY_A, eos_token_id=[7, 9, 11])
    cfg, spec = resolve(d)
    assert cfg.eos_token_ids == (7, 9, 11) and spec.eos_token_ids == (7, 9, 11)
    assert cfg.to_dict()["eos_token_id"] == [7, 9, 11]
    assert resolve(dict(TINY_A, eos_token_id=None))[1].eos_token_ids == ()


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
    assert spec.layers[1].parts["mixer"].kind == "attention" and spec.layers[1].parts["ffn"].kind == "swiglu"
    assert spec.layers[1].parts["mixer"].name == "self_attn" and spec.layers[1].block == "pre_norm"
    assert spec.layers[0].parts["mixer"].params["position"]["theta"] == 500000.0
    assert spec.lm_head.params["tied_to"] == "model.embed_tokens" and spec.embedding.name == "model.embed_tokens"
    assert "tied_to" not in resolve(TINY_A)[1].lm_head.params
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


def test_sizes_a_kernel_refuses_are_refused_when_the_model_is_built():
    """bfloat16 products move 16-byte vectors: a width that is no multiple of 8 fails at build time,
    with the part and the size named; float32 takes it."""
    from tiny_llm_amd.kernels.ops import KernelError
    odd = dict(TINY_A, hidden_size=68, num_attention_heads=2, num_key_value_heads=1, head_dim=34)
    _, spec = resolve(odd)
    Decoder(spec, "float32", "cpu")
    with pytest.raises(KernelError) as e:
        Decoder(spec, "bfloat16", "cpu")
    assert "68" in str(e.value) and "multiple of 8" in str(e.value)
    _, spec = resolve(dict(TINY_A, intermediate_size=177))
    with pytest.raises(KernelError) as e:
        Decoder(spec, "bfloat16", "cpu")
    assert "intermediate_size = 177" in str(e.value)
    _, spec = resolve(dict(TINY_A, hidden_size=1056, num_attention_heads=4, num_key_value_heads=4, head_dim=264))
    with pytest.raises(KernelError) as e:
        Decoder(spec, "float32", "cpu")
    assert "head_dim 264" in str(e.value)


def test_cache_pool_is_sized_by_configuration_or_by_free_memory():
    from tiny_llm_amd.engine.loading import plan_cache_blocks
    e = EngineConfig(kv_block_size=16, max_num_seqs=4)
    assert plan_cache_blocks(EngineConfig(num_kv_blocks=7), 100, 1000, 10 ** 9) == 7
    assert plan_cache_blocks(EngineConfig(kv_block_size=16, max_cache_tokens=100), 100, 1000, 10 ** 9) == 7
    assert plan_cache_blocks(e, 100, 1000, None) == 4 * 7                      # worst case: can never run out
    assert plan_cache_blocks(e, 100, 1000, 10 ** 9) == 28                      # memory is plenty
    assert plan_cache_blocks(e, 100, 1000, 20000) == 18                        # 0.9 of 20000 bytes / 1000
    with pytest.raises(MemoryError):
        plan_cache_blocks(e, 100, 1000, 500)


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


def test_tensors_set_by_hand_shadow_the_file(tmp_path):
    # (ref) tests/weight_managers/test_safetensors.cpp:31-56: a missing name throws; set, read back,
    # set again with another shape, read back; tensors of the file stay readable
    from tiny_llm_amd.weights import Checkpoint
    save_file({"embedding": torch.arange(6, dtype=torch.float32).reshape(2, 3),
               "attention": torch.arange(10, 14, dtype=torch.float32).reshape(2, 2)},
              str(tmp_path / "model.safetensors"))
    ck = Checkpoint(str(tmp_path))
    with pytest.raises(SafetensorsError):
        ck.get("random")
    mine = torch.tensor([100.0, 200.0])
    ck.set_tensor("random", mine)
    mine[0] = -1.0                                   # the checkpoint holds a copy
    assert ck.info("random") == (torch.float32, (2,)) and ck.get("random").tolist() == [100.0, 200.0]
    ck.set_tensor("random", torch.tensor([[50.0, 100.0]]))
    assert ck.info("random") == (torch.float32, (1, 2)) and ck.get("random").tolist() == [[50.0, 100.0]]
    ck.set_tensor("attention", torch.zeros(3))       # shadows the file's tensor
    assert ck.get("attention").tolist() == [0, 0, 0] and ck.get("embedding").tolist() == [[0, 1, 2], [3, 4, 5]]
    assert sorted(ck.names()) == ["attention", "embedding", "random"]
    with pytest.raises(ValueError):
        ck.set_tensor("empty", torch.zeros(0))


def test_loading_through_a_checkpoint_with_tensors_set_by_hand(tmp_path):
    from tiny_llm_amd.weights import Checkpoint
    folder = write_random_model(str(tmp_path), TINY_A, seed=5)
    ck = Checkpoint(folder)
    ck.set_tensor("model.norm.weight", torch.full((64,), 3.0))
    dec = _specs(TINY_A)
    load_weights(dec, ck)
    assert dec.final_norm.weight.tolist() == [3.0] * 64
    ck.set_tensor("model.norm.weight", torch.full((63,), 3.0))
    with pytest.raises(WeightLoadError) as e:
        load_weights(_specs(TINY_A), ck)
    assert e.value.wrong_shape == [("model.norm.weight", (64,), (63,))]


def test_sharded_folder_loads_like_a_single_file(tmp_path):
    """model.safetensors.index.json and its shards (how larger checkpoints are published)."""
    single = write_random_model(str(tmp_path / "single"), TINY_B, seed=4, norm_std=0.1)
    f = SafetensorsFile(os.path.join(single, "model.safetensors"))
    names = f.names()
    shard_dir = tmp_path / "sharded"
    shard_dir.mkdir()
    weight_map = {}
    for i in range(3):
        part = {n: f.get(n).clone() for n in names[i::3]}
        fname = f"model-{i + 1:05d}-of-00003.safetensors"
        save_file(part, str(shard_dir / fname))
        weight_map.update({n: fname for n in part})
    json.dump({"metadata": {}, "weight_map": weight_map}, open(shard_dir / "model.safetensors.index.json", "w"))
    json.dump(json.load(open(os.path.join(single, "config.json"))), open(shard_dir / "config.json", "w"))
    a, b = _specs(TINY_B), _specs(TINY_B)
    load_weights(a, single)
    load_weights(b, str(shard_dir))
    for pa, pb in zip(a.parts(), b.parts()):
        for k, v in vars(pa).items():
            if isinstance(v, torch.Tensor):
                assert torch.equal(v, getattr(pb, k)), (pa.prefix, k)
    os.remove(shard_dir / "model-00002-of-00003.safetensors")
    with pytest.raises(SafetensorsError):
        load_weights(_specs(TINY_B), str(shard_dir))


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
    assert dec.layers[1].by_role["ffn"].w_gate_up.shape == (2 * 176, 64)
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


def test_seeded_numbers_are_normal_and_a_pure_function_of_seed_name_and_index():
    from tiny_llm_amd.weights.loader import _standard_normal_host, tensor_key
    z = torch.from_numpy(_standard_normal_host(tensor_key(1, "x"), 1 << 20)).double()
    assert abs(float(z.mean())) < 5e-3 and abs(float(z.std()) - 1) < 5e-3
    assert abs(float((z ** 4).mean()) - 3) < 0.05 and abs(float((z ** 3).mean())) < 0.02
    assert abs(float((z.abs() < 1).double().mean()) - 0.6827) < 3e-3
    # element i does not depend on how many elements are made, nor on the chunking
    a = _standard_normal_host(tensor_key(1, "x"), 1000, chunk=64)
    assert torch.equal(torch.from_numpy(a), z[:1000].float())
    # a norm weight: 1 + norm_std * z, each operation rounded to float32
    n = random_tensor(WeightSpec("n.weight", (50,), role="vector", init="ones"), 9, 0.02, 0.1)
    zz = torch.from_numpy(_standard_normal_host(tensor_key(9, "n.weight"), 50))
    assert torch.equal(n, zz * torch.tensor(0.1, dtype=torch.float32) + 1.0)
    assert torch.equal(random_tensor(WeightSpec("n.weight", (50,), role="vector", init="ones"), 9, 0.02, 0.0),
                       torch.ones(50))


def test_tied_head_is_not_stored_and_shares_the_table(tmp_path):
    folder = write_random_model(str(tmp_path), TINY_B, seed=1, norm_std=0.1)
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    assert "lm_head.weight" not in f
    dec = _specs(TINY_B)
    load_weights(dec, folder)
    assert dec.lm_head.weight.data_ptr() == dec.embedding.weight.data_ptr()
    norm = f.get("model.layers.2.input_layernorm.weight")
    assert 0.03 < float(norm.std()) < 0.3 and abs(float(norm.mean()) - 1) < 0.1


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_all_resident_weights_lie_in_one_slab(cfg, tmp_path):
    """Every tensor a part holds after loading is a view of ONE allocation, at a 256-byte boundary;
    a tied head is the embedding's view, not a second copy; nothing is left outside; and the values
    are the file's (fused, interleaved or as they came)."""
    folder = write_random_model(str(tmp_path), cfg, seed=4, norm_std=0.1)
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    dec = _specs(cfg)
    load_weights(dec, folder)
    slab = dec.weight_slab
    lo, hi = slab.buffer.data_ptr(), slab.buffer.data_ptr() + slab.buffer.numel()
    held, seen = 0, set()
    for part in dec.parts():
        for name, t in vars(part).items():
            if not isinstance(t, torch.Tensor):
                continue
            assert lo <= t.data_ptr() and t.data_ptr() + t.numel() * t.element_size() <= hi, (part.prefix, name)
            assert (t.data_ptr() - lo) % 256 == 0
            if t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                held += t.numel() * t.element_size()
    assert slab.outside == 0
    stored = sum(f.get(n).numel() * 4 for n in f.names())       # float32 on this path
    assert held == stored and slab.used >= held and slab.buffer.numel() < stored + 256 * (len(f.names()) + 64)
    if cfg.get("tie_word_embeddings"):
        assert dec.lm_head.weight.data_ptr() == dec.embedding.weight.data_ptr()
    layer = dec.layers[1]
    q, k, v = (f.get(f"model.layers.1.self_attn.{n}_proj.weight") for n in "qkv")
    assert torch.equal(layer.by_role["mixer"].w_qkv, torch.cat([q, k, v]))
    gate, up = f.get("model.layers.1.mlp.gate_proj.weight"), f.get("model.layers.1.mlp.up_proj.weight")
    assert torch.equal(layer.by_role["ffn"].w_gate_up[0::2], gate) and torch.equal(layer.by_role["ffn"].w_gate_up[1::2], up)
    assert torch.equal(dec.final_norm.weight, f.get("model.norm.weight"))


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
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)      # the architecture says: ignorable
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


def test_what_may_be_ignored_is_the_architectures_to_say(tmp_path):
    import dataclasses
    folder = write_random_model(str(tmp_path), TINY_A, seed=5)
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.get(n).clone() for n in f.names()}
    del f
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    save_file(tensors, path)
    _, spec = resolve(TINY_A)
    assert spec.ignorable_tensors == ("*.rotary_emb.inv_freq",)
    load_weights(Decoder(spec, "float32", "cpu"), folder)
    strict = dataclasses.replace(spec, ignorable_tensors=())
    with pytest.raises(WeightLoadError) as e:
        load_weights(Decoder(strict, "float32", "cpu"), folder)
    assert e.value.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]


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
