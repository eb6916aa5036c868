"""SwiGLU feed-forward: down( silu(gate(h)) * up(h) ), residual add folded in.

Reference: tiny_llm/parser/llama_parser.cpp:225-255 (gate, SiLU in place, up,
multiply, down, add), tiny_llm/ops/cuda/silu.cu:10 (x / (1 + exp(-x))).  Gate and
up weights are concatenated on load into one [2I, H] matrix.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import FeedForward, WeightSpec, register_feed_forward


class SwiGLU(FeedForward):
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, intermediate_size: int):
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        p, H, I = self.prefix, self.hidden_size, self.intermediate_size
        return [WeightSpec(f"{p}.gate_proj.weight", (I, H)), WeightSpec(f"{p}.up_proj.weight", (I, H)),
                WeightSpec(f"{p}.down_proj.weight", (H, I))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        p = self.prefix
        self.w_gate_up = torch.cat([tensors[f"{p}.gate_proj.weight"], tensors[f"{p}.up_proj.weight"]],
                                   dim=0).contiguous()
        self.w_down = tensors[f"{p}.down_proj.weight"].contiguous()

    def forward(self, h, ctx, residual):
        T = h.shape[0]
        gate_up = torch.empty((T, 2 * self.intermediate_size), dtype=self.dtype, device=h.device)
        ops.linear(h, self.w_gate_up, gate_up)
        z = torch.empty((T, self.intermediate_size), dtype=self.dtype, device=h.device)
        ops.silu_mul(gate_up, z)
        return ops.linear(z, self.w_down, residual, residual)


register_feed_forward("swiglu", SwiGLU)
