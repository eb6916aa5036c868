"""The Llama architecture as data: LlamaConfig -> ModelSpec.

Layer order and part placement follow tiny_llm/parser/llama_parser.cpp:194-271:
embedding; per layer input_layernorm -> self_attn -> +residual ->
post_attention_layernorm -> mlp -> +residual; model.norm; lm_head.  Weight-name
prefixes are the checkpoint's (llama_parser.cpp:181, 199-265).
"""
from __future__ import annotations

from ..config.llama import LlamaConfig
from ..config.registry import register_architecture
from ..config.spec import LayerSpec, ModelSpec, PartSpec, PlanEntry


def build_llama_spec(cfg: LlamaConfig) -> ModelSpec:
    norm = lambda: PartSpec("rmsnorm", {"hidden_size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    layers = []
    for i in range(cfg.num_hidden_layers):
        layers.append(LayerSpec(
            prefix=f"model.layers.{i}",
            block="pre_norm",
            mixer_norm=norm(),
            mixer=PartSpec("attention", {
                "hidden_size": cfg.hidden_size,
                "num_heads": cfg.num_attention_heads,
                "num_kv_heads": cfg.num_key_value_heads,
                "head_dim": cfg.head_dim,
                "max_position": cfg.max_position_embeddings,
                "position": {"kind": "rotary", "head_dim": cfg.head_dim, "theta": cfg.rope_theta,
                             "max_position": cfg.max_position_embeddings},
            }),
            ffn_norm=norm(),
            ffn=PartSpec("swiglu", {"hidden_size": cfg.hidden_size,
                                    "intermediate_size": cfg.intermediate_size}),
        ))
    return ModelSpec(
        architecture="LlamaForCausalLM",
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        max_position=cfg.max_position_embeddings,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size}),
        layers=tuple(layers),
        plan=tuple(PlanEntry(i) for i in range(cfg.num_hidden_layers)),
        final_norm=norm(),
        lm_head=PartSpec("lm_head", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size,
                                     "tied": cfg.tie_word_embeddings}),
        eos_token_id=cfg.eos_token_id,
    )


register_architecture
from ..config.spec import LayerSpec, ModelSpec, PartSpec, PlanEntry


def build_llama_spec(cfg: LlamaConfig) -> ModelSpec:
    norm = lambda: PartSpec("rmsnorm", {"hidden_size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    layers = []
    for i in range(cfg.num_hidden_layers):
        layers.append(LayerSpec(
            prefix=f"model.layers.{i}",
            block="pre_norm",
            mixer_norm=norm(),
            mixer=PartSpec("attention", {
                "hidden_size": cfg.hidden_size,
                "num_heads": cfg.num_attention_heads,
                "num_kv_heads": cfg.num_key_value_heads,
                "head_dim": cfg.head_dim,
                "max_position": cfg.max_position_embeddings,
                "position": {"kind": "rotary", "head_dim": cfg.head_dim, "theta": cfg.rope_theta,
                             "max_position": cfg.max_position_embeddings},
            }),
            ffn_norm=norm(),
            ffn=PartSpec("swiglu", {"hidden_size": cfg.hidden_size,
                                    "intermediate_size": cfg.intermediate_size}),
        ))
    return ModelSpec(
        architecture="LlamaForCausalLM",
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        max_position=cfg.max_position_embeddings,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size}),
        layers=tuple(layers),
        plan=tuple(PlanEntry(i) for i in range(cfg.num_hidden_layers)),
        final_norm=norm(),
        lm_head=PartSpec("lm_head", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size,
                                     "tied": cfg.tie_word_embeddings}),
        eos_token_id=cfg.eos_token_id,
    )


# Weight-name parts that the Llama layer kinds use below a layer's prefix.
LLAMA_PART_NAMES = {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                    "ffn_norm": "post_attention_layernorm", "ffn": "mlp"}

register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, build_llama_spec)
