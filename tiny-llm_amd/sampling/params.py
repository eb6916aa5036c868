"""Per-request generation options, named as the reference's `Pipeline::apply` arguments
and command-line flags (tiny_llm/pipeline/pipeline.hpp:24-29, main.cpp:7-19)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class SamplingParams:
    max_new_tokens: int = 256
    do_sample: bool = True          # False: greedy (first maximum)
    temperature: float = 0.7
    top_k: int = 50                 # 0 keeps every token (the reference's 0 empties the set)
    top_p: float = 0.95             # 1 keeps every token
    seed: Optional[int] = None      # None: drawn from the engine's seed and the request's number
    ignore_eos: bool = False

    def __post_init__(self):
        if self.max_new_tokens < 0:
            raise ValueError("max_new_tokens must not be negative")
        if self.do_sample:
            # the reference divides by the temperature and throws on 0
            # (tiny_llm/ops/cpu/arithmetic.cpp:75-78)
            if not (self.temperature > 0):
                raise ValueError("temperature must be positive when sampling")
            if not (0.0 <= self.top_p <= 1.0):
                raise ValueError("top_p must lie in [0, 1]")   # sort_processors.cpp:82-89
            if self.top_k < 0:
                raise ValueError("top_k must not be negative")

    @classmethod
    def greedy(cls, max_new_tokens: int = 256, **kw) -> "SamplingParams":
        return cls(max_new_tokens=max_new_tokens, do_sample=False, **kw)
