"""Block arrangements.  "pre_norm" is Llama's: x + mixer(norm(x)), then
x + ffn(norm(x)) (tiny_llm/parser/llama_parser.cpp:194-255)."""
from __future__ import annotations

from .base import Block, register_block


class PreNormBlock(Block):
    roles = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "ffn": "feed_forward"}

    def __init__(self, parts):
        super().__init__(parts)
        self.mixer_norm, self.mixer = parts["mixer_norm"], parts["mixer"]
        self.ffn_norm, self.ffn = parts["ffn_norm"], parts["ffn"]

    def forward(self, x, ctx, caches, states):
        return self.forward_chained(x, ctx, caches, states)[0]

    @property
    def first_norm(self):
        """The norm that reads this block's input, for whoever writes that input."""
        return self.mixer_norm if getattr(self.mixer, "accepts_lazy_norm", False) else None

    def forward_chained(self, x, ctx, caches, states, prepared=None, next_norm=None):
        """As `forward`, between neighbours: `prepared` is this block's first norm as prepared by the
        product that wrote x (or None); `next_norm` is the norm that will read this block's result
        (or None).  Returns (x, that norm prepared or None)."""
        h = self._normed(self.mixer_norm, self.mixer, x, prepared)
        ffn_norm = self.ffn_norm if getattr(self.ffn, "accepts_lazy_norm", False) else None
        x, prep = self._run(self.mixer, (h, ctx, caches.get("mixer"), states.get("mixer"), x), ffn_norm)
        h = self._normed(self.ffn_norm, self.ffn, x, prep)
        return self._run(self.ffn, (h, ctx, x), next_norm)

    @staticmethod
    def _run(part, args, next_norm):
        if next_norm is not None and getattr(part, "prepares_next_norm", False):
            out = part.forward(*args, next_norm=next_norm)
            return out if isinstance(out, tuple) else (out, None)
        return part.forward(*args), None

    @staticmethod
    def _normed(norm, consumer, x, prepared=None):
        # a consumer that says so may receive the norm unevaluated and fuse it into its first product
        if getattr(consumer, "accepts_lazy_norm", False) and hasattr(norm, "lazy"):
            return norm.lazy(x, prepared=prepared) if prepared is not None else norm.lazy(x)
        return norm.forward(x)


register_block("pre_norm", PreNormBlock)
