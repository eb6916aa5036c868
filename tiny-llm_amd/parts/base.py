"""Interfaces of the parts a layer is made of, and the registries that name them.

A part is built from a PartSpec's parameters alone: it knows its own sizes and
constants and nothing about the model it sits in.  The generic decoder
(models/decoder.py) looks parts up here by name, layer by layer, so one model
may mix kinds.  Tests and other architectures add kinds with the `register_*`
functions; no framework file changes.

Calling conventions
-------------------
* The residual stream `x` is float32 [tokens, hidden].
* A norm maps x (float32) to the activation type of the engine.
* A mixer and a feed-forward receive the normed activations `h` and the
  residual, and return `residual + f(h)` as float32 (writing into `residual`
  is allowed); `add_to_residual` does that for parts that do not fuse it.
* A part with `prepares_next_norm = True` also takes `next_norm=` (the norm that will read its
  result, or None) and may return `(residual, prepared)`: it has prepared that norm in its last
  product (`project_into_residual`).  Nothing else has to know about this.
* A mixer additionally receives the step context (who is in the batch, where
  each token sits), its view of the paged cache (or None) and its per-request
  state tensor [slots, ...] (or None).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch


# ------------------------------------------------------------------ declarations
@dataclass(frozen=True)
class WeightSpec:
    """One checkpoint tensor a part needs.

    role: "matrix" - operand of a matrix product, takes the engine's element type;
          "vector" - norm weights and the like: engine type, except that a tensor
                     stored in 32 bits stays in 32 bits;
          "table"  - integer tables, kept as int32.
    init: how random-weights mode fills it ("normal" | "ones" | "around_one").
    alias_of: a tensor to use when the file does not hold `name` (tied weights).
    """
    name: str
    shape: Tuple[int, ...]
    role: str = "matrix"
    init: str = "normal"
    alias_of: Optional[str] = None


@dataclass(frozen=True)
class CacheTensor:
    """One paged tensor of a cache: per token it keeps `shape` elements, and a page is
    [block_size tokens] put at axis `token_axis` of that shape (keys of 4 heads of 64 are
    shape (4, 64) with token_axis 1: pages [4, block_size, 64]; one latent vector of 96 per token is
    shape (96,) with token_axis 0: pages [block_size, 96])."""
    name: str
    shape: Tuple[int, ...]
    token_axis: int = 0

    def page_shape(self, block_size: int) -> Tuple[int, ...]:
        s = list(self.shape)
        s.insert(self.token_axis, block_size)
        return tuple(s)


@dataclass(frozen=True)
class CacheSpec:
    """What a mixer keeps per token, as a list of paged tensors.
    kind "full" keeps every position, "window" the last `window` positions.
    Layers whose specs are equal share one block-id space and one block table per request."""
    tensors: Tuple[CacheTensor, ...]
    kind: str = "full"
    window: int = 0

    @classmethod
    def keys_and_values(cls, num_kv_heads: int, head_dim: int, kind: str = "full", window: int = 0) -> "CacheSpec":
        """The usual attention cache: tensors "k" and "v", pages [kv_heads, block_size, head_dim]."""
        t = (int(num_kv_heads), int(head_dim))
        return cls((CacheTensor("k", t, 1), CacheTensor("v", t, 1)), kind, int(window))

    def group_key(self):
        return (self.kind, self.window, self.tensors)


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size: one tensor of `shape` per live request."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerCache:
    """A mixer's view of the paged cache for one run of its layer: the tensors its CacheSpec
    names, each [blocks, *page_shape]."""
    tensors: Dict[str, torch.Tensor]
    group: int                 # which block table / slot mapping of the context applies
    write: bool = True         # False: the run reads a cache that another run fills

    @property
    def k(self) -> torch.Tensor:
        return self.tensors["k"]

    @property
    def v(self) -> torch.Tensor:
        return self.tensors["v"]


class Part:
    """Base of every part: declares weights, receives them, computes."""

    # True if `forward` only enqueues device work whose shape depends on nothing but the step's
    # capacities (no host reads of step data, no host loops over requests): such a part may be
    # captured in a HIP graph.  Parts defined elsewhere default to False: their layer then runs
    # eagerly between the graphs of the layers around it, with the step's host copies in `ctx`.
    graph_safe = False

    def __init__(self, prefix: str, dtype: torch.dtype, device: torch.device):
        self.prefix = prefix
        self.dtype = dtype
        self.device = device

    def weights(self) -> List[WeightSpec]:
        return []

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Receives the device tensors named by `weights()` (full names)."""

    def cache_spec(self) -> Optional[CacheSpec]:
        """Paged per-token memory this part needs (None: none)."""
        return None

    def state_spec(self) -> Optional[StateSpec]:
        """Per-request memory of fixed size this part needs (None: none)."""
        return None


class Embedding(Part):
    """Token ids [T] (int32) -> the residual stream, float32 [T, hidden]."""

    def forward(self, tokens: torch.Tensor, ctx=None) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    """Normed activations at the wanted rows -> float32 logits [rows, vocab]."""

    def forward(self, h) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """How positions enter a mixer.  `rotary_tables()` returns
    (cos, sin, rotary_dim) for encodings that rotate queries and keys, or None."""

    def rotary_tables(self):
        return None


class Mixer(Part):
    def forward(self, h: torch.Tensor, ctx, cache: Optional[LayerCache], state: Optional[torch.Tensor],
                residual: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, ctx, residual: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Block:
    """An arrangement of a layer's parts around the residual stream.

    `roles` names the parts the arrangement wants and the registry each is looked up in
    ("norm", "mixer", "feed_forward", ...: the keys of REGISTRIES).  The decoder builds them and
    hands them over as a dict; `caches` and `states` in `forward` are dicts by role that hold an
    entry for every part that declared a cache or a state."""

    roles: Dict[str, str] = {}

    def __init__(self, parts: Dict[str, Part]):
        missing = [r for r in self.roles if r not in parts]
        extra = [r for r in parts if r not in self.roles]
        if missing or extra:
            raise ValueError(f"{type(self).__name__} takes the parts {sorted(self.roles)}; "
                             f"missing {missing}, not taken {extra}")
        self._parts = dict(parts)

    def parts(self) -> List[Part]:
        return list(self._parts.values())

    def forward(self, x, ctx, caches, states):
        raise NotImplementedError


def project_into_residual(z: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, next_norm=None):
    """residual += z @ w.T, the last product of a mixer or feed-forward.  Returns
    (residual, prepared): when `next_norm` (the norm that will read the result) can be prepared by
    this very product (few rows, bfloat16), `prepared` is what its `lazy()` takes; else None."""
    from ..kernels import ops
    bufs = None
    if next_norm is not None and hasattr(next_norm, "hand_off_buffers") and residual.is_contiguous():
        bufs = next_norm.hand_off_buffers(residual.shape[0], z.shape[1], residual.device)
    if bufs is not None and z.dtype == torch.bfloat16 and bufs[1].shape == residual.shape:
        ops.linear_handoff(z, w, residual, residual, emit=bufs)
        return residual, (bufs[1], bufs[2])
    return ops.linear(z, w, residual, residual), None


def add_to_residual(residual: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """residual += y in float32, for parts whose last kernel does not fuse the add."""
    from ..kernels import ops
    return ops.add_residual(residual, y.contiguous())


# -------------------------------------------------------------------- registries
class Registry:
    def __init__(self, what: str):
        self.what = what
        self._items: Dict[str, Callable[..., Any]] = {}

    def register(self, name: str, factory: Callable[..., Any], *, replace: bool = False) -> None:
        if name in self._items and not replace:
            raise ValueError(f"{self.what} {name!r} is already registered")
        self._items[name] = factory

    def unregister(self, name: str) -> None:
        self._items.pop(name, None)

    def get(self, name: str) -> Callable[..., Any]:
        if name not in self._items:
            raise KeyError(f"no {self.what} named {name!r}; known: {', '.join(sorted(self._items))}")
        return self._items[name]

    def names(self):
        return sorted(self._items)


EMBEDDINGS = Registry("embedding")
HEADS = Registry("output head")
NORMS = Registry("norm")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block arrangement")


# a block's roles and the model's own parts name their registry by these keys
REGISTRIES = {"embedding": EMBEDDINGS, "head": HEADS, "norm": NORMS, "mixer": MIXERS,
              "feed_forward": FEED_FORWARDS, "position_encoding": POSITION_ENCODINGS}


def register_embedding(name, factory, **kw): EMBEDDINGS.register(name, factory, **kw)
def register_head(name, factory, **kw): HEADS.register(name, factory, **kw)
def register_norm(name, factory, **kw): NORMS.register(name, factory, **kw)
def register_mixer(name, factory, **kw): MIXERS.register(name, factory, **kw)
def register_feed_forward(name, factory, **kw): FEED_FORWARDS.register(name, factory, **kw)
def register_position_encoding(name, factory, **kw): POSITION_ENCODINGS.register(name, factory, **kw)
def register_block(name, factory, **kw): BLOCKS.register(name, factory, **kw)
