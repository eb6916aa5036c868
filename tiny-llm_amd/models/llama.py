"""The Llama architecture as data: LlamaConfig -> ModelSpec.

Layer order and part placement follow tiny_llm/parser/llama_parser.cpp:194-271:
embedding; per layer input_layernorm -> self_attn -> +residual ->
post_attention_layernorm -> mlp -> +residual; model.norm; lm_head.  Weight-name
prefixes are the checkpoint's (llama_parser.cpp:181, 199-265).
"""
from __future__ import annotations

from ..config.llama import LlamaConfig
from ..config.registry import register_architecture
from ..config.spec import ModelSpec, PartSpec, PlanEntry, pre_norm_layer

# Weight-name component of each role below a layer's prefix.
LLAMA_PART_NAMES = {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                    "ffn_norm": "post_attention_layernorm", "ffn": "mlp"}

# Published checkpoints of this family carry the rotary frequencies as a buffer; no part reads it.
LLAMA_IGNORABLE = ("*.rotary_emb.inv_freq",)


def build_llama_spec(cfg: LlamaConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"hidden_size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    attention = PartSpec("attention", {
        "hidden_size": cfg.hidden_size,
        "num_heads": cfg.num_attention_heads,
        "num_kv_heads": cfg.num_key_value_heads,
        "head_dim": cfg.head_dim,
        "position": {"kind": "rotary", "head_dim": cfg.head_dim, "theta": cfg.rope_theta,
                     "max_position": cfg.max_position_embeddings},
    })
    ffn = PartSpec("swiglu", {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size})
    layers = tuple(pre_norm_layer(f"model.layers.{i}", norm, attention, norm, ffn, LLAMA_PART_NAMES)
                   for i in range(cfg.num_hidden_layers))
    sizes = {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size}
    head = dict(sizes, tied_to="model.embed_tokens") if cfg.tie_word_embeddings else sizes
    return ModelSpec(
        architecture="LlamaForCausalLM",
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        max_position=cfg.max_position_embeddings,
        embedding=PartSpec("token_embedding", sizes, "model.embed_tokens"),
        layers=layers,
        plan=tuple(PlanEntry(i) for i in range(cfg.num_hidden_layers)),
        final_norm=norm.named("model.norm"),
        lm_head=PartSpec("lm_head", head, "lm_head"),
        eos_token_ids=cfg.eos_token_ids,
        ignorable_tensors=LLAMA_IGNORABLE,
    )


register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, build_llama_spec)
