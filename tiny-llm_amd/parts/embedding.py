"""Token embedding (a row gather, no scale: tiny_llm/ops/cuda/embedding.cu:10-29)
and the output head (logits = xn W^T at the wanted rows only:
tiny_llm/ops/cuda/gemm_q1_helper.cu:99-124).  A tied head uses the embedding
table; the reference never reads `tie_word_embeddings`."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import Embedding, Head, WeightSpec, register_embedding, register_head
from .norm import LazyNorm


class TokenEmbedding(Embedding):
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, vocab_size: int, hidden_size: int):
        super().__init__(prefix, dtype, device)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        return [WeightSpec(f"{self.prefix}.weight", (self.vocab_size, self.hidden_size))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[f"{self.prefix}.weight"].contiguous()

    def forward(self, tokens: torch.Tensor, ctx=None) -> torch.Tensor:
        out = ops.scratch("residual", (tokens.numel(), self.hidden_size), torch.float32, tokens.device)
        return ops.embedding(tokens, self.weight, out)


class LMHead(Head):
    graph_safe = True
    accepts_lazy_norm = True

    def __init__(self, prefix, dtype, device, *, vocab_size: int, hidden_size: int, tied_to: str = None):
        super().__init__(prefix, dtype, device)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.tied_to = tied_to          # weight prefix of the embedding whose table this head shares
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        self.weight: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        alias = f"{self.tied_to}.weight" if self.tied_to else None
        return [WeightSpec(f"{self.prefix}.weight", (self.vocab_size, self.hidden_size), alias_of=alias)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[f"{self.prefix}.weight"].contiguous()

    def forward(self, h) -> torch.Tensor:
        """h: activations [n, H], or a LazyNorm whose norm rides in the product."""
        if isinstance(h, LazyNorm):
            out = torch.empty((h.num_rows, self.vocab_size), dtype=torch.float32, device=h.x.device)
            return h.linear(self.weight, out)
        out = torch.empty((h.shape[0], self.vocab_size), dtype=torch.float32, device=h.device)
        return ops.linear(h, self.weight, out)


register_embedding("token_embedding", TokenEmbedding)
register_head("lm_head", LMHead)
