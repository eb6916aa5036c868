"""Rotary position encoding: the angle tables and the pairing.

theta[p, i] = p * base^(-i / (rotary_dim/2)), computed in float64 and rounded to
float32 cos / sin tables of shape [max_position, rotary_dim/2], as the reference
does (tiny_llm/ops/cuda/rope.cu:12-24).  The rotation itself (the reference's
rotate-half pairing (i, i + rotary_dim/2), rope.cu:46-54) is fused with the cache
write in the attention mixer's kernels; this part owns the constants:
(theta, rotary_dim, pairing, scaling).

pairing  "half" (the reference's) or "interleaved" (pair i is the dims 2i, 2i + 1).
scaling  None, or {"kind": "linear", "factor": f}: positions are divided by f before the
         angles are taken (the table changes, nothing else).  Other kinds are refused by name.
"""
from __future__ import annotations

from typing import Dict, Tuple

import torch

from .base import PositionEncoding, register_position_encoding

# Angle tables by (rotary_dim, theta, max_position, position factor, device): the layers of a model share one pair.
_TABLES: Dict[Tuple, Tuple[torch.Tensor, torch.Tensor]] = {}

PAIRINGS = ("half", "interleaved")
SCALINGS = ("linear",)


def angle_tables(rotary_dim: int, theta: float, max_position: int, device,
                 position_factor: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """float32 (cos, sin) [max_position, rotary_dim / 2] of theta[p, i] = (p / position_factor) *
    base^(-i / (rotary_dim / 2)), computed in float64 on the host (tiny_llm/ops/cuda/rope.cu:12-24,
    which has no factor)."""
    key = (int(rotary_dim), float(theta), int(max_position), float(position_factor), str(torch.device(device)))
    if key not in _TABLES:
        half = rotary_dim // 2
        idx = torch.arange(half, dtype=torch.float64)
        inv_freq = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -idx / half)
        pos = torch.arange(max_position, dtype=torch.float64)
        if position_factor != 1.0:
            pos = pos / float(position_factor)
        ang = pos[:, None] * inv_freq[None, :]
        _TABLES[key] = (torch.cos(ang).to(torch.float32).contiguous().to(device),
                        torch.sin(ang).to(torch.float32).contiguous().to(device))
    return _TABLES[key]


class RotaryEmbedding(PositionEncoding):
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, head_dim: int, theta: float, max_position: int,
                 rotary_dim: int = None, pairing: str = "half", scaling: dict = None):
        super().__init__(prefix, dtype, device)
        if pairing not in PAIRINGS:
            raise ValueError(f"rotary pairing {pairing!r} is not built; known: {', '.join(PAIRINGS)}")
        self.pairing = pairing
        factor = 1.0
        if scaling is not None:
            kind = dict(scaling).get("kind")
            if kind not in SCALINGS:
                raise ValueError(f"rotary scaling {kind!r} is not built; known: {', '.join(SCALINGS)}")
            factor = float(scaling["factor"])
            if not factor > 0:
                raise ValueError("the factor of linear rotary scaling must be positive")
        self.position_factor = factor
        self.head_dim = int(head_dim)
        self.rotary_dim = int(head_dim if rotary_dim is None else rotary_dim)
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= self.head_dim):
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        self.theta = float(theta)
        self.max_position = int(max_position)
        self.cos, self.sin = angle_tables(self.rotary_dim, self.theta, self.max_position, device, factor)

    def rotary_tables(self):
        return self.cos, self.sin, self.rotary_dim


class NoPositionEncoding(PositionEncoding):
    graph_safe = True

    def __init__(self, prefix, dtype, device, **_):
        super().__init__(prefix, dtype, device)


register_position_encoding("rotary", RotaryEmbedding)
register_position_encoding("none", NoPositionEncoding)
