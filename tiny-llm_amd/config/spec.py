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
    """One part by registry name, with every size and constant it needs.

    `name` is where its weights live: for the parts of a layer the component below the layer's
    prefix ("self_attn" -> "model.layers.3.self_attn.*"), for the model's own parts (embedding,
    final norm, output head) the whole prefix ("model.embed_tokens")."""
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)
    name: str = ""

    def named(self, name: str) -> "PartSpec":
        return PartSpec(self.kind, self.params, name)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: parts by role, and the block arrangement that runs them.

    The roles are the arrangement's own ("pre_norm" has mixer_norm, mixer, ffn_norm and ffn; an
    arrangement registered elsewhere may have others); the arrangement says which registry each
    role is looked up in."""
    prefix: str                 # weight-name prefix, e.g. "model.layers.3"
    block: str                  # arrangement, e.g. "pre_norm"
    parts: Mapping[str, PartSpec]


def pre_norm_layer(prefix: str, mixer_norm: PartSpec, mixer: PartSpec, ffn_norm: PartSpec, ffn: PartSpec,
                   names: Optional[Mapping[str, str]] = None) -> LayerSpec:
    """The usual layer: x + mixer(norm(x)), then x + ffn(norm(x)).  `names` gives the weight-name
    component of each role; a part that already has a name keeps it, the others get the role."""
    names = dict(names or {})
    parts = {}
    for role, ps in (("mixer_norm", mixer_norm), ("mixer", mixer), ("ffn_norm", ffn_norm), ("ffn", ffn)):
        parts[role] = ps if ps.name else ps.named(names.get(role, role))
    return LayerSpec(prefix, "pre_norm", parts)


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
    embedding: PartSpec          # its `name` is the whole weight prefix
    layers: Tuple[LayerSpec, ...]
    plan: Tuple[PlanEntry, ...]
    final_norm: PartSpec
    lm_head: PartSpec
    eos_token_ids: Tuple[int, ...] = ()
    # glob patterns of tensors that checkpoints of this architecture carry and no part needs
    ignorable_tensors: Tuple[str, ...] = ()

    def validate(self) -> None:
        n = len(self.layers)
        if not self.plan:
            raise ValueError("a model needs at least one plan entry")
        for what in ("embedding", "final_norm", "lm_head"):
            if not getattr(self, what).name:
                raise ValueError(f"the model's {what} needs a weight prefix (PartSpec.name)")
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
