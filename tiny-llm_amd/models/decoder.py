"""The generic decoder: a ModelSpec made into parts, and the forward pass of one step.

It knows no architecture.  Every part (embedding, the parts of each layer, final norm,
output head) is looked up by kind in the part registries and built from its PartSpec;
weight prefixes come from the spec.  The decoder collects what the parts declare
(weights, cache needs, per-request state) and runs the plan: a list of layer runs, in
which a layer may appear twice or read the cache of an earlier run.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..config.spec import LayerSpec, ModelSpec, PartSpec
from ..parts import BLOCKS, REGISTRIES, CacheSpec, LayerCache, Part, StateSpec, WeightSpec

TORCH_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}

# (plan entry, role of the part within its layer): who owns a cache or a state
Owner = Tuple[int, str]


def build_part(category: str, spec: PartSpec, prefix: str, dtype, device) -> Part:
    return REGISTRIES[category].get(spec.kind)(prefix, dtype, device, **dict(spec.params))


class Layer:
    def __init__(self, spec: LayerSpec, dtype, device):
        arrangement = BLOCKS.get(spec.block)
        roles = getattr(arrangement, "roles", None)
        if not roles:
            raise ValueError(f"block arrangement {spec.block!r} does not say which parts it takes (`roles`)")
        unknown = [r for r in spec.parts if r not in roles]
        if unknown:
            raise ValueError(f"layer {spec.prefix}: arrangement {spec.block!r} has no role {unknown}; "
                             f"it takes {sorted(roles)}")
        self.by_role: Dict[str, Part] = {}
        for role, category in roles.items():
            if role not in spec.parts:
                raise ValueError(f"layer {spec.prefix}: arrangement {spec.block!r} needs a part for role {role!r}")
            ps = spec.parts[role]
            self.by_role[role] = build_part(category, ps, f"{spec.prefix}.{ps.name or role}", dtype, device)
        self.block = arrangement(self.by_role)

    def parts(self) -> List[Part]:
        return list(self.by_role.values())

    @property
    def mixer(self):
        """The layer's part of role "mixer" (None in an arrangement without that role)."""
        return self.by_role.get("mixer")


class Decoder:
    def __init__(self, spec: ModelSpec, dtype: str = "bfloat16", device="cuda:0"):
        spec.validate()
        self.spec = spec
        self.dtype = TORCH_DTYPES[dtype] if isinstance(dtype, str) else dtype
        self.device = torch.device(device)
        self.embedding = build_part("embedding", spec.embedding, spec.embedding.name, self.dtype, self.device)
        self.layers: List[Layer] = [Layer(ls, self.dtype, self.device) for ls in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm, spec.final_norm.name, self.dtype, self.device)
        self.lm_head = build_part("head", spec.lm_head, spec.lm_head.name, self.dtype, self.device)
        # cache and state views by role, per plan entry; attached by the runner once the pools exist
        self.caches: List[Dict[str, LayerCache]] = [{} for _ in spec.plan]
        self.states: List[Dict[str, torch.Tensor]] = [{} for _ in spec.plan]
        self._graph_safe: Optional[bool] = None
        self._graph_runs: Optional[List[tuple]] = None

    # ---------------------------------------------------------------- declarations
    def parts(self) -> List[Part]:
        out = [self.embedding]
        for l in self.layers:
            out.extend(l.parts())
        out.extend([self.final_norm, self.lm_head])
        return out

    @property
    def graph_safe(self) -> bool:
        """True if every part (and every part's position encoding) may be captured in a HIP graph.
        (Asked at every step; the parts do not change once the decoder is built.)"""
        if self._graph_safe is None:
            parts = self.parts()
            parts += [getattr(p, "position", None) for p in parts]
            self._graph_safe = all(p.graph_safe for p in parts if p is not None)
        return self._graph_safe

    def weight_specs(self) -> List[WeightSpec]:
        specs: List[WeightSpec] = []
        for p in self.parts():
            specs.extend(p.weights())
        return specs

    def cache_specs(self) -> Dict[Owner, CacheSpec]:
        """The caches the plan's runs own (a run that reads another run's cache owns none)."""
        out: Dict[Owner, CacheSpec] = {}
        for i, e in enumerate(self.spec.plan):
            if e.cache_of is not None:
                continue
            for role, part in self.layers[e.layer].by_role.items():
                cs = part.cache_spec()
                if cs is not None:
                    out[(i, role)] = cs
        return out

    def cache_readers(self) -> Dict[Owner, Owner]:
        """Runs that read the cache of an earlier run: reader -> owner."""
        out: Dict[Owner, Owner] = {}
        for i, e in enumerate(self.spec.plan):
            if e.cache_of is None:
                continue
            for role, part in self.layers[e.layer].by_role.items():
                if part.cache_spec() is not None:
                    out[(i, role)] = (e.cache_of, role)
        return out

    def state_specs(self) -> Dict[Owner, StateSpec]:
        out: Dict[Owner, StateSpec] = {}
        for i, e in enumerate(self.spec.plan):
            for role, part in self.layers[e.layer].by_role.items():
                ss = part.state_spec()
                if ss is not None:
                    out[(i, role)] = ss
        return out

    # --------------------------------------------------------------------- compute
    # The pass in stages: stage 0 embeds the tokens, stage 1 + i is entry i of the plan, the last
    # one is the final norm and the head.  A step runs all of them in one call; a captured step of
    # a model that holds a part which may not be captured runs them in runs of stages, the
    # capturable runs as HIP graphs and the others eagerly between them.
    @property
    def num_stages(self) -> int:
        return len(self.spec.plan) + 2

    def stage_graph_safe(self, stage: int) -> bool:
        if stage == 0:
            parts = [self.embedding]
        elif stage == self.num_stages - 1:
            parts = [self.final_norm, self.lm_head]
        else:
            parts = self.layers[self.spec.plan[stage - 1].layer].parts()
        parts = parts + [getattr(p, "position", None) for p in parts]
        return all(p.graph_safe for p in parts if p is not None)

    def graph_runs(self) -> List[tuple]:
        """The stages in runs that may be captured and runs that may not: (capturable, first, last)
        with stages first .. last - 1, in order."""
        if self._graph_runs is None:
            runs: List[tuple] = []
            for st in range(self.num_stages):
                safe = self.stage_graph_safe(st)
                if runs and runs[-1][0] == safe:
                    runs[-1] = (safe, runs[-1][1], st + 1)
                else:
                    runs.append((safe, st, st + 1))
            self._graph_runs = runs
        return self._graph_runs

    def forward(self, ctx) -> torch.Tensor:
        """Runs the tokens of `ctx` through the plan; float32 logits at ctx.logit_rows."""
        return self.run_stages(ctx, 0, self.num_stages, None)

    def run_stages(self, ctx, first: int, last: int, x: Optional[torch.Tensor]) -> torch.Tensor:
        """Stages first .. last - 1.  `x` is the residual stream the stage before `first` left (None
        for stage 0).  Returns the residual stream, or, behind the last stage, the logits.  A norm is
        handed from one block to the next only inside one call."""
        n = self.num_stages
        plan = self.spec.plan
        wants_logits = ctx.logit_rows is not None and ctx.logit_rows.numel() > 0
        # a head that says so may receive the final norm unevaluated and fuse it into its product
        lazy_head = hasattr(self.final_norm, "lazy") and getattr(self.lm_head, "accepts_lazy_norm", False)
        if first == 0:
            x = self.embedding.forward(ctx.tokens, ctx)
        # A block may prepare the norm that reads its result (the next block's first norm, or the
        # final norm) in its last product; `prepared` carries that from one block to the next.
        prepared = None
        for st in range(max(first, 1), min(last, n - 1)):
            i = st - 1
            block = self.layers[plan[i].layer].block
            if not hasattr(block, "forward_chained"):
                x, prepared = block.forward(x, ctx, self.caches[i], self.states[i]), None
                continue
            next_norm = None
            if st + 1 < last:                    # what reads this block's result runs in this call
                if i + 1 < len(plan):
                    nxt = self.layers[plan[i + 1].layer].block
                    next_norm = getattr(nxt, "first_norm", None) if hasattr(nxt, "forward_chained") else None
                else:
                    next_norm = self.final_norm if wants_logits and lazy_head else None
            x, prepared = block.forward_chained(x, ctx, self.caches[i], self.states[i], prepared, next_norm)
        if last < n:
            return x
        if not wants_logits:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=x.device)
        norm = self.final_norm
        rows = None if getattr(ctx, "logits_all_rows", False) else ctx.logit_rows
        if lazy_head:
            h = norm.lazy(x, rows, prepared=prepared) if prepared is not None else norm.lazy(x, rows)
        else:
            h = norm.forward(x, rows)
        return self.lm_head.forward(h)
