"""Sampling settings.  The token itself is chosen on the device at the end of the step
(`kernels.ops.sample`, called by `engine.step`): greedy rows take the first maximum; sampling
rows run the reference's chain temperature -> top-k -> top-p -> multinomial
(tiny_llm/pipeline/pipeline.cpp:156-164) in one kernel.  The uniform number of a row comes from
(seed, counter): the request's seed and the position of the token being chosen, so a request's
tokens do not depend on what else is in the batch or on how its prompt was cut."""
from .params import SamplingParams
