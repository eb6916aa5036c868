"""RMSNorm: y = w * x / sqrt(mean(x^2) + eps), statistics in float32.

Reference: tiny_llm/ops/cuda/norm.cu:29-48 (weight applied before the division,
plain `w`, not `1 + w`); placed by tiny_llm/parser/llama_parser.cpp:198-203,
219-224, 258-263.  Unlike the reference (norm.cu:66-85) any width is taken.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import Norm, WeightSpec, register_norm


class LazyNorm:
    """A norm that has not run yet: (x, weight, eps).  A consumer that can fuse the norm into its
    first product takes the fields; any other calls `materialize()`."""

    def __init__(self, norm: "RMSNorm", x: torch.Tensor, rows: Optional[torch.Tensor] = None):
        self.norm, self.x, self.rows = norm, x, rows
        self.weight, self.eps = norm.weight, norm.eps

    @property
    def num_rows(self) -> int:
        return self.x.shape[0] if self.rows is None else self.rows.numel()

    def materialize(self) -> torch.Tensor:
        return self.norm.forward(self.x, self.rows)


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, eps: float, init: str = "ones"):
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self.init = init
        self.weight: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        return [WeightSpec(f"{self.prefix}.weight", (self.hidden_size,), role="vector", init=self.init)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[f"{self.prefix}.weight"].contiguous()

    def lazy(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None):
        """In bfloat16 the norm rides in the consumer's first product (`ops.linear_norm`)."""
        if self.dtype == torch.bfloat16 and self.hidden_size % 8 == 0:
            return LazyNorm(self, x, rows)
        return self.forward(x, rows)

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.hidden_size), dtype=self.dtype, device=x.device)
        return ops.rmsnorm(x, self.weight, self.eps, out, rows)


register_norm("rmsnorm", RMSNorm)
