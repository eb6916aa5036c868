"""A model as data: which parts make each layer, and in which order layers run.

Nothing here computes.  An architecture's builder turns its typed configuration
into a ModelSpec; the generic decoder (models/decoder.py) instantiates the named
parts from the part registries and runs the plan.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part by registry name, with every size and constant it needs."""
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a mixer and a feed-forward, each behind its norm, in a block."""
    prefix: str                 # weight-name prefix, e.g. "model.layers.3"
    block: str                  # arrangement of the four parts, e.g. "pre_norm"
    mixer_norm: PartSpec
    mixer: PartSpec
    ffn_norm: PartSpec
    ffn: PartSpec
    # weight-name component of each part below `prefix`
    part_names: Mapping[str, str] = field(default_factory=lambda: {
        "mixer_norm": "input_layernorm", "mixer": "self_attn",
        "ffn_norm": "post_attention_layernorm", "ffn": "mlp"})


@dataclass(frozen=True)
class PlanEntry:
    """One run of a layer.  `cache_of` names an earlier plan entry whose cache
    this run reads instead of keeping its own (it then writes nothing)."""
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_position: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    plan: Tuple[PlanEntry, ...]
    final_norm: PartSpec
    lm_head: PartSpec
    eos_token_id: Optional[int] = None

    def validate(self) -> None:
        n = len(self.layers)
        if not self.plan:
            raise ValueError("a model needs at least one plan entry")
        for i, e in enumerate(self.plan):
            if not (0 <= e.layer < n):
                raise ValueError(f"plan entry {i} names layer {e.layer}, model has {n}")
            if e.cache_of is not None:
                if not (0 <= e.cache_of < i):
                    raise ValueError(
                        f"plan entry {i} reads the cache of entry {e.cache_of}, "
                        "which must be an earlier entry")
                if self.plan[e.cache_of].cache_of is not None:
                    raise ValueError(
                        f"plan entry {i} reads the cache of entry {e.cache_of}, "
                        "which itself has no cache of its own")
