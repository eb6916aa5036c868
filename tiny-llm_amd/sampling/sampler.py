"""Token selection for a batch of logits rows, on the device.

Greedy rows take the first maximum; sampling rows run the reference's chain
temperature -> top-k -> top-p -> multinomial (tiny_llm/pipeline/pipeline.cpp:156-164)
in one kernel.  The uniform number of a row comes from (seed, counter): the request's
seed and the position of the token being chosen, so a request's tokens do not depend
on what else is in the batch or on how its prompt was cut.
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from ..kernels import ops
from .params import SamplingParams


class Sampler:
    def __init__(self, device):
        self.device = device

    def __call__(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
                 counters: Sequence[int]) -> List[int]:
        """logits float32 [n, vocab] on the device -> n token ids on the host."""
        n = logits.shape[0]
        out = torch.empty(n, dtype=torch.int32, device=logits.device)
        if all(not p.do_sample for p in params):
            ops.sample(logits, out)
            return out.cpu().tolist()
        host = torch.empty((5, n), dtype=torch.float64)
        for i, p in enumerate(params):
            host[0, i] = p.temperature if p.do_sample else 0.0
            host[1, i] = p.top_k
            host[2, i] = p.top_p
            host[4, i] = counters[i]
        temperature = host[0].to(torch.float32).to(logits.device)
        top_k = host[1].to(torch.int32).to(logits.device)
        top_p = host[2].to(torch.float32).to(logits.device)
        seed_t = torch.tensor([s & 0x7FFFFFFFFFFFFFFF for s in seeds], dtype=torch.int64, device=logits.device)
        ctr = host[4].to(torch.int32).to(logits.device)
        ops.sample(logits, out, temperature, top_k, top_p, seed_t, ctr)
        return out.cpu().tolist()
