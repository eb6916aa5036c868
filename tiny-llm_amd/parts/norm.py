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
    first product takes the fields; any other calls `materialize()`.

    `prepared` = (operand, sumsq): the product that wrote x has already written
    operand = bf16(weight * x) and the sums of x^2 over groups of columns
    (`ops.linear_handoff`), so the consumer's product needs no pass over x at all."""

    def __init__(self, norm: "RMSNorm", x: torch.Tensor, rows: Optional[torch.Tensor] = None, prepared=None):
        self.norm, self.x, self.rows = norm, x, rows
        self.weight, self.eps = norm.weight, norm.eps
        self.prepared = prepared

    def linear(self, w: torch.Tensor, out: torch.Tensor, epilogue: Optional[str] = None) -> torch.Tensor:
        """out = norm(x)[rows] @ w.T (then the epilogue), by the cheapest route there is."""
        if self.x.dtype == torch.float32 and w.dtype == torch.float32:
            # true float32: the norm inside the few-row product's kernel (measured on whole steps: up
            # to 16 rows it saves time), or as two kernels that give the same bits: norm_weight * x
            # and the rows' factors, then the product with the factor applied to its sums
            # (a product so wide that a workgroup owns several column tiles takes the two kernels too)
            if (self.rows is None and self.x.shape[0] <= RMSNorm.F32_FUSED_ROWS
                    and ops.linear_norm_f32_ok(self.x.shape[0], w.shape[0], self.x.shape[1], self.x.stride(0))
                    and ops.linear_f32_col_tiles(self.x.shape[0], w.shape[0], self.x.shape[1]) == 1):
                return ops.linear_norm_f32(self.x, self.weight, self.eps, w, out, epilogue=epilogue)
            h, inv_rms = ops.norm_prescale_f32(self.x, self.weight, self.eps, self.rows)
            return ops.linear(h, w, out, epilogue=epilogue, row_scale=inv_rms)
        if self.prepared is not None and (self.num_rows <= ops.FEW_ROWS or self.rows is None):
            operand, sumsq = self.prepared
            return ops.linear_handoff(operand, w, out, epilogue=epilogue, rows=self.rows,
                                      prepared=(sumsq, self.eps, self.x.shape[1]))
        return ops.linear_norm(self.x, self.weight, self.eps, w, out, rows=self.rows, epilogue=epilogue)

    @property
    def num_rows(self) -> int:
        return self.x.shape[0] if self.rows is None else self.rows.numel()

    def materialize(self) -> torch.Tensor:
        return self.norm.forward(self.x, self.rows)


class RMSNorm(Norm):
    graph_safe = True
    F32_FUSED_ROWS = 16      # measured on whole steps: beyond, the norm's own kernel is as fast or faster

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

    def lazy(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None, prepared=None):
        """The norm rides in the consumer's first product: in bfloat16 always (`ops.linear_norm`), in
        float32 for at most 16 rows (`ops.linear_norm_f32`); more rows, or gathered rows, get the
        norm as a row factor of the product (`ops.norm_prescale_f32`), which gives the same bits."""
        if self.dtype == torch.bfloat16 and self.hidden_size % 8 == 0:
            return LazyNorm(self, x, rows, prepared)
        if self.dtype == torch.float32 and self.weight.dtype == torch.float32:
            return LazyNorm(self, x, rows, None)
        return self.forward(x, rows)

    def hand_off_buffers(self, n_rows: int, inner: int, device):
        """(weight, operand, sumsq) for a product (inner size `inner`) that writes this norm's input
        and can prepare the norm on the way (`ops.linear_handoff`), or None where that does not apply."""
        if not ops.can_hand_off(n_rows, self.hidden_size, inner, self.dtype):
            return None
        # still read by the next product while the product after that writes its own: three in turn
        operand = ops.scratch("handoff_operand", (n_rows, self.hidden_size), torch.bfloat16, device, rotate=3)
        sumsq = ops.scratch("handoff_sumsq", (n_rows, ops.handoff_parts(n_rows, self.hidden_size, inner)),
                            torch.float32, device, rotate=3)
        return self.weight, operand, sumsq

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.numel()
        # two in turn: a block's second norm is computed while nothing reads its first any more, but
        # the final norm's rows must not alias what a consumer still holds
        out = ops.scratch("normed", (n, self.hidden_size), self.dtype, x.device, rotate=2)
        return ops.rmsnorm(x, self.weight, self.eps, out, rows)


register_norm("rmsnorm", RMSNorm)
