"""SwiGLU feed-forward: down( silu(gate(h)) * up(h) ), residual add folded in.

Reference: tiny_llm/parser/llama_parser.cpp:225-255 (gate, SiLU in place, up,
multiply, down, add), tiny_llm/ops/cuda/silu.cu:10 (x / (1 + exp(-x))).  Gate and
up weights are interleaved row by row on load into one [2I, H] matrix, and the
SiLU-gate runs in the epilogue of that one product on its float32 accumulators:
the [T, 2I] intermediate of the reference's four kernels is never written.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .norm import LazyNorm
from .base import FeedForward, WeightSpec, project_into_residual, register_feed_forward


class SwiGLU(FeedForward):
    graph_safe = True
    accepts_lazy_norm = True
    prepares_next_norm = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, intermediate_size: int):
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        ops.check_linear_sizes(dtype, self.intermediate_size, f"{prefix}: intermediate_size")
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        p, H, I = self.prefix, self.hidden_size, self.intermediate_size
        return [WeightSpec(f"{p}.gate_proj.weight", (I, H)), WeightSpec(f"{p}.up_proj.weight", (I, H)),
                WeightSpec(f"{p}.down_proj.weight", (H, I))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        p = self.prefix
        gate, up = tensors[f"{p}.gate_proj.weight"], tensors[f"{p}.up_proj.weight"]
        # rows interleaved (gate_0, up_0, gate_1, up_1, ...): a product's epilogue then sees each
        # pair side by side and writes silu(gate) * up directly
        self.w_gate_up = torch.stack([gate, up], dim=1).reshape(2 * self.intermediate_size,
                                                                self.hidden_size).contiguous()
        self.w_down = tensors[f"{p}.down_proj.weight"].contiguous()

    def forward(self, h, ctx, residual, next_norm=None):
        T, dev = residual.shape[0], residual.device
        z = ops.scratch("ffn_gated", (T, self.intermediate_size), self.dtype, dev)
        if isinstance(h, LazyNorm):
            h.linear(self.w_gate_up, z, epilogue="swiglu")
        else:
            ops.linear(h, self.w_gate_up, z, epilogue="swiglu")
        out, prepared = project_into_residual(z, self.w_down, residual, next_norm)
        return out if next_norm is None else (out, prepared)


register_feed_forward("swiglu", SwiGLU)
