"""Shared test material: the tiny configurations, model folders, comparisons."""
import json
import os

import torch

# Where the reference's checkout lies (its tests' fixtures are read from there, never run): beside
# this repository unless TINY_LLM_REFERENCE says otherwise.  Tests that need a fixture skip without it.
REFERENCE = os.environ.get("TINY_LLM_REFERENCE") or os.path.join(
    os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))), "reference")
REFERENCE_DATA = os.path.join(REFERENCE, "tests", "datas")

# Two tiny configurations of the architecture that differ in every size and option.
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "intermediate_size": 176, "vocab_size": 251, "rope_theta": 10000.0, "rms_norm_eps": 1e-5,
    "max_position_embeddings": 640, "tie_word_embeddings": False, "hidden_act": "silu",
    "attention_bias": False, "rope_scaling": None, "initializer_range": 0.02, "eos_token_id": 2,
    "torch_dtype": "float32",
}
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
    "head_dim": 32, "intermediate_size": 200, "vocab_size": 517, "rope_theta": 500000.0,
    "rms_norm_eps": 1e-6, "max_position_embeddings": 1024, "tie_word_embeddings": True,
    "hidden_act": "silu", "attention_bias": False, "rope_scaling": None, "initializer_range": 0.05,
    "eos_token_id": 5, "torch_dtype": "float32",
}
# A third one with heads of 128 and as many kv heads as heads (the shape of attention of the larger Llamas).
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 256, "num_attention_heads": 2, "num_key_value_heads": 2,
    "head_dim": 128, "intermediate_size": 352, "vocab_size": 333, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5, "max_position_embeddings": 512, "tie_word_embeddings": False,
    "hidden_act": "silu", "attention_bias": False, "rope_scaling": None, "initializer_range": 0.03,
    "eos_token_id": 3, "torch_dtype": "float32",
}
# A fourth whose heads are no multiple of 16 wide (the general attention kernel) and do not add up to
# the hidden size; pages of four tokens.
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 136, "num_attention_heads": 6, "num_key_value_heads": 2,
    "head_dim": 40, "intermediate_size": 232, "vocab_size": 409, "rope_theta": 7000.0,
    "rms_norm_eps": 3e-6, "max_position_embeddings": 384, "tie_word_embeddings": False,
    "hidden_act": "silu", "attention_bias": False, "rope_scaling": None, "initializer_range": 0.04,
    "eos_token_id": 7, "torch_dtype": "float32",
}
# engine-side options that go with them
ENGINE_A = {"kv_block_size": 16}
ENGINE_B = {"kv_block_size": 8}
ENGINE_C = {"kv_block_size": 32}
ENGINE_D = {"kv_block_size": 4}
INIT_A = {"std": 0.02, "norm_std": 0.0}
INIT_B = {"std": 0.05, "norm_std": 0.1}
INIT_C = {"std": 0.03, "norm_std": 0.05}
INIT_D = {"std": 0.04, "norm_std": 0.2}

CONFIGS = {"A": (TINY_A, ENGINE_A, INIT_A), "B": (TINY_B, ENGINE_B, INIT_B), "C": (TINY_C, ENGINE_C, INIT_C),
           "D": (TINY_D, ENGINE_D, INIT_D)}


def make_folder(tmp_path, cfg, seed=0, std=0.02, norm_std=0.0, dtype="float32", sharpen=4.0):
    """Writes a model folder with seeded weights.  q and k projections are scaled by
    `sharpen` so that attention is far from uniform and a misplaced key changes the logits."""
    from tiny_llm_amd.weights import write_random_model, save_file
    from safetensors import safe_open
    folder = str(tmp_path)
    write_random_model(folder, cfg, seed=seed, std=std, norm_std=norm_std, dtype=dtype)
    if sharpen and sharpen != 1.0:
        path = os.path.join(folder, "model.safetensors")
        tensors = {}
        with safe_open(path, "pt") as f:
            for k in f.keys():
                t = f.get_tensor(k).clone()
                if k.endswith("q_proj.weight") or k.endswith("k_proj.weight"):
                    t = (t.float() * sharpen).to(t.dtype)
                tensors[k] = t
        save_file(tensors, path + ".tmp")
        os.replace(path + ".tmp", path)
    return folder


def read_weights(folder, round_to=None):
    """Weights of a folder as float64, read with the safetensors library (not the engine's
    reader); `round_to=torch.bfloat16` rounds them as the serving path does."""
    from safetensors import safe_open
    out = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        for k in f.keys():
            t = f.get_tensor(k)
            if round_to is not None and t.dim() >= 2:
                t = t.to(round_to)
            out[k] = t.to(torch.float64)
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return out, cfg


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """max |got - ref| over max |ref|, per comparison (rows share one scale)."""
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


def random_tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
