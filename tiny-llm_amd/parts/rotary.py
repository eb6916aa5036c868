"""Rotary position encoding: the angle tables.

theta[p, i] = p * base^(-i / (rotary_dim/2)), computed in float64 and rounded to
float32 cos / sin tables of shape [max_position, rotary_dim/2], as the reference
does (tiny_llm/ops/cuda/rope.cu:12-24).  The rotation itself (rotate-half
pairing (i, i + rotary_dim/2), rope.cu:46-54) is fused with the cache write in
the attention mixer's kernel; this part only owns the constants.
"""
from __future__ import annotations

from typing import Dict, Tuple

import torch

from .base import PositionEncoding, register_position_encoding

# Angle tables by (rotary_dim, theta, max_position, device): the layers of a model share one pair.
_TABLES: Dict[Tuple, Tuple[torch.Tensor, torch.Tensor]] = {}


def angle_tables(rotary_dim: int, theta: float, max_position: int, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """float32 (cos, sin) [max_position, rotary_dim / 2] of theta[p, i] = p * base^(-i / (rotary_dim / 2)),
    computed in float64 on the host (tiny_llm/ops/cuda/rope.cu:12-24)."""
    key = (int(rotary_dim), float(theta), int(max_position), str(torch.device(device)))
    if key not in _TABLES:
        half = rotary_dim // 2
        idx = torch.arange(half, dtype=torch.float64)
        inv_freq = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -idx / half)
        ang = torch.arange(max_position, dtype=torch.float64)[:, None] * inv_freq[None, :]
        _TABLES[key] = (torch.cos(ang).to(torch.float32).contiguous().to(device),
                        torch.sin(ang).to(torch.float32).contiguous().to(device))
    return _TABLES[key]


class RotaryEmbedding(PositionEncoding):
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, head_dim: int, theta: float, max_position: int,
                 rotary_dim: int = None):
        super().__init__(prefix, dtype, device)
        self.head_dim = int(head_dim)
        self.rotary_dim = int(head_dim if rotary_dim is None else rotary_dim)
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= self.head_dim):
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        self.theta = float(theta)
        self.max_position = int(max_position)
        self.cos, self.sin = angle_tables(self.rotary_dim, self.theta, self.max_position, device)

    def rotary_tables(self):
        return self.cos, self.sin, self.rotary_dim


class NoPositionEncoding(PositionEncoding):
    graph_safe = True

    def __init__(self, prefix, dtype, device, **_):
        super().__init__(prefix, dtype, device)


register_position_encoding("rotary", RotaryEmbedding)
register_position_encoding("none", NoPositionEncoding)
