"""The generic decoder: a ModelSpec made into parts, and the forward pass of one step.

It does not know Llama.  It instantiates the parts each LayerSpec names, collects
what they declare (weights, cache needs, per-request state), and runs the plan:
a list of layer runs, in which a layer may appear twice or read the cache of an
earlier run.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..config.spec import ModelSpec
from ..parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, CacheSpec, LayerCache, StateSpec, WeightSpec)
from ..parts.embedding import LMHead, TokenEmbedding

TORCH_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


class Layer:
    def __init__(self, spec, dtype, device):
        p = spec.prefix
        part_names = spec.part_names
        mk = lambda reg, ps, sub: reg.get(ps.kind)(f"{p}.{part_names[sub]}", dtype, device, **dict(ps.params))
        self.mixer_norm = mk(NORMS, spec.mixer_norm, "mixer_norm")
        self.mixer = mk(MIXERS, spec.mixer, "mixer")
        self.ffn_norm = mk(NORMS, spec.ffn_norm, "ffn_norm")
        self.ffn = mk(FEED_FORWARDS, spec.ffn, "ffn")
        self.block = BLOCKS.get(spec.block)(self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    def parts(self):
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]


class Decoder:
    def __init__(self, spec: ModelSpec, dtype: str = "bfloat16", device="cuda:0"):
        spec.validate()
        self.spec = spec
        self.dtype = TORCH_DTYPES[dtype] if isinstance(dtype, str) else dtype
        self.device = torch.device(device)
        e = dict(spec.embedding.params)
        self.embedding = TokenEmbedding("model.embed_tokens", self.dtype, self.device, **e)
        self.layers: List[Layer] = [Layer(ls, self.dtype, self.device) for ls in spec.layers]
        self.final_norm = NORMS.get(spec.final_norm.kind)("model.norm", self.dtype, self.device,
                                                          **dict(spec.final_norm.params))
        h = dict(spec.lm_head.params)
        tied = h.pop("tied", False)
        self.lm_head = LMHead("lm_head", self.dtype, self.device, tied_to="model.embed_tokens" if tied else None, **h)
        # cache and state views are attached by the runner once the pools exist
        self.caches: List[Optional[LayerCache]] = [None] * len(spec.plan)
        self.states: List[Optional[torch.Tensor]] = [None] * len(spec.plan)

    # ---------------------------------------------------------------- declarations
    def parts(self):
        out = [self.embedding]
        for l in self.layers:
            out.extend(l.parts())
        out.extend([self.final_norm, self.lm_head])
        return out

    @property
    def graph_safe(self) -> bool:
        """True if every part (and every mixer's position encoding) may be captured in a HIP graph."""
        parts = self.parts() + [getattr(l.mixer, "position", None) for l in self.layers]
        return all(p.graph_safe for p in parts if p is not None)

    def weight_specs(self) -> List[WeightSpec]:
        specs: List[WeightSpec] = []
        for p in self.parts():
            specs.extend(p.weights())
        return specs

    def cache_specs(self) -> List[Optional[CacheSpec]]:
        """Per plan entry: the cache it owns (None if it has none or reads another's)."""
        out = []
        for e in self.spec.plan:
            out.append(None if e.cache_of is not None else self.layers[e.layer].mixer.cache_spec())
        return out

    def state_specs(self) -> List[Optional[StateSpec]]:
        return [self.layers[e.layer].mixer.state_spec() for e in self.spec.plan]

    # --------------------------------------------------------------------- compute
    def forward(self, ctx) -> torch.Tensor:
        """Runs the tokens of `ctx` through the plan; float32 logits at ctx.logit_rows."""
        x = self.embedding.forward(ctx.tokens)
        wants_logits = ctx.logit_rows is not None and ctx.logit_rows.numel() > 0
        plan = self.spec.plan
        # A block may prepare the norm that reads its result (the next block's first norm, or the
        # final norm) in its last product; `prepared` carries that from one block to the next.
        prepared = None
        for i, e in enumerate(plan):
            block = self.layers[e.layer].block
            if not hasattr(block, "forward_chained"):
                x, prepared = block.forward(x, ctx, self.caches[i], self.states[i]), None
                continue
            if i + 1 < len(plan):
                nxt = self.layers[plan[i + 1].layer].block
                next_norm = getattr(nxt, "first_norm", None) if hasattr(nxt, "forward_chained") else None
            else:
                next_norm = self.final_norm if wants_logits and hasattr(self.final_norm, "lazy") else None
            x, prepared = block.forward_chained(x, ctx, self.caches[i], self.states[i], prepared, next_norm)
        if not wants_logits:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=x.device)
        norm = self.final_norm
        if hasattr(norm, "lazy"):
            h = norm.lazy(x, ctx.logit_rows, prepared=prepared) if prepared is not None else norm.lazy(x, ctx.logit_rows)
        else:
            h = norm.forward(x, ctx.logit_rows)
        return self.lm_head.forward(h)
