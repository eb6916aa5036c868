"""Block arrangements.  "pre_norm" is Llama's: x + mixer(norm(x)), then
x + ffn(norm(x)) (tiny_llm/parser/llama_parser.cpp:194-255)."""
from __future__ import annotations

from .base import Block, register_block


class PreNormBlock(Block):
    def forward(self, x, ctx, cache, state):
        h = self._normed(self.mixer_norm, self.mixer, x)
        x = self.mixer.forward(h, ctx, cache, state, x)
        h = self._normed(self.ffn_norm, self.ffn, x)
        return self.ffn.forward(h, ctx, x)

    @staticmethod
    def _normed(norm, consumer, x):
        # a consumer that says so may receive the norm unevaluated and fuse it into its first product
        if getattr(consumer, "accepts_lazy_norm", False) and hasattr(norm, "lazy"):
            return norm.lazy(x)
        return norm.forward(x)


register_block("pre_norm", PreNormBlock)
