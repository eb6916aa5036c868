"""Typed configuration of the Llama architecture, read from config.json keys.

The reference indexes the raw json at every use site and gives no key a default
(tiny_llm/parser/llama_parser.cpp:165-267, tiny_llm/pipeline/pipeline.cpp:47-82).
Here the keys are read once into a frozen dataclass, defaulted where the key is
optional in published Llama checkpoints, and validated; parts never see json.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, asdict
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that this architecture cannot run."""


_REQUIRED = (
    "vocab_size",
    "hidden_size",
    "intermediate_size",
    "num_hidden_layers",
    "num_attention_heads",
)


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    hidden_act: str
    attention_bias: bool
    mlp_bias: bool
    eos_token_ids: Tuple[int, ...]       # every id that ends a request (config.json may list several)
    bos_token_id: Optional[int]
    torch_dtype: str
    initializer_range: float
    architectures: tuple = ("LlamaForCausalLM",)

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "LlamaConfig":
        missing = [k for k in _REQUIRED if k not in d or d[k] is None]
        if missing:
            raise ConfigError(f"config.json lacks required keys: {', '.join(missing)}")
        nq = int(d["num_attention_heads"])
        if nq <= 0:
            raise ConfigError("num_attention_heads must be positive")
        hidden = int(d["hidden_size"])
        nkv = d.get("num_key_value_heads")
        nkv = nq if nkv is None else int(nkv)
        head_dim = d.get("head_dim")
        if head_dim is None:
            # The reference fixes head_dim = hidden_size / num_attention_heads
            # (llama_parser.cpp:173); the key, where present, overrides it.
            if hidden % nq:
                raise ConfigError(
                    f"hidden_size {hidden} is not divisible by num_attention_heads {nq} "
                    "and config.json gives no head_dim")
            head_dim = hidden // nq
        eos = d.get("eos_token_id")
        if eos is None:
            eos = ()
        elif not isinstance(eos, (list, tuple)):
            eos = (eos,)
        arch = d.get("architectures") or ["LlamaForCausalLM"]
        cfg = cls(
            vocab_size=int(d["vocab_size"]),
            hidden_size=hidden,
            intermediate_size=int(d["intermediate_size"]),
            num_hidden_layers=int(d["num_hidden_layers"]),
            num_attention_heads=nq,
            num_key_value_heads=nkv,
            head_dim=int(head_dim),
            max_position_embeddings=int(d.get("max_position_embeddings", 2048)),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-6)),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            hidden_act=str(d.get("hidden_act", "silu")),
            attention_bias=bool(d.get("attention_bias", False)),
            mlp_bias=bool(d.get("mlp_bias", False)),
            eos_token_ids=tuple(int(e) for e in eos),
            bos_token_id=None if d.get("bos_token_id") is None else int(d["bos_token_id"]),
            torch_dtype=str(d.get("torch_dtype", "float32")),
            initializer_range=float(d.get("initializer_range", 0.02)),
            architectures=tuple(arch),
        )
        cfg._validate(d)
        return cfg

    @classmethod
    def from_json(cls, path: str) -> "LlamaConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path, "r", encoding="utf-8") as f:
            return cls.from_dict(json.load(f))

    # --------------------------------------------------------------- validation
    def _validate(self, raw: Mapping[str, Any]) -> None:
        # Same refusals as the reference (llama_parser.cpp:165-169): no biases,
        # no rope scaling, SiLU only.
        if self.attention_bias or self.mlp_bias:
            raise ConfigError("attention_bias / mlp_bias = true is not supported")
        if raw.get("rope_scaling") is not None:
            raise ConfigError("rope_scaling must be null")
        if self.hidden_act != "silu":
            raise ConfigError(f"hidden_act must be 'silu', got {self.hidden_act!r}")
        for k in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                  "num_key_value_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, k) <= 0:
                raise ConfigError(f"{k} must be positive, got {getattr(self, k)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even for rotary positions")
        if not (self.rms_norm_eps > 0):
            raise ConfigError("rms_norm_eps must be positive")
        if not (self.rope_theta > 0):
            raise ConfigError("rope_theta must be positive")

    @property
    def eos_token_id(self) -> Optional[int]:
        """The first end-of-sequence id (None if the checkpoint names none)."""
        return self.eos_token_ids[0] if self.eos_token_ids else None

    # ---------------------------------------------------------------- writing
    def to_dict(self) -> dict:
        d = asdict(self)
        eos = d.pop("eos_token_ids")
        d["eos_token_id"] = None if not eos else (eos[0] if len(eos) == 1 else list(eos))
        d["architectures"] = list(self.architectures)
        d["model_type"] = "llama"
        d["rope_scaling"] = None
        return d
