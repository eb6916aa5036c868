"""Block arrangements.  "pre_norm" is Llama's: x + mixer(norm(x)), then
x + ffn(norm(x)) (tiny_llm/parser/llama_parser.cpp:194-255)."""
from __future__ import annotations

from .base import Block, register_block


class PreNormBlock(Block):
    def forward(self, x, ctx, cache, state):
        h = self.mixer_norm.forward(x)
        x = self.mixer.forward(h, ctx, cache, state, x)
        h = self.ffn_norm.forward(x)
        return self.ffn.forward(h, ctx, x)


register_block("pre_norm", PreNormBlock)
