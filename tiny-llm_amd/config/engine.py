"""Engine-side sizes: what the cache pool, the batch and the scheduler may use.

The reference has `PipelineConfig{model_type, dtype, device, paged, max_requests}`
(tiny_llm/pipeline/pipeline.hpp:14-21) and a literal page size of 32
(tiny_llm/runtime/cuda/cuda_runtime.cpp:16); its pool is sized for the worst case
so it can never run out (cuda_runtime.cpp:510-515).  Here every size is a field.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

DTYPES = {"float32": "float32", "fp32": "float32", "f32": "float32",
          "bfloat16": "bfloat16", "bf16": "bfloat16"}


@dataclass
class EngineConfig:
    dtype: str = "bfloat16"            # "bfloat16" (serving) or "float32" (true 32-bit)
    kv_block_size: int = 16            # tokens per cache page
    num_kv_blocks: Optional[int] = None  # pages per cache group; None = from max_cache_tokens
    max_cache_tokens: Optional[int] = None  # None too: worst case, capped by free device memory
    cache_memory_fraction: float = 0.9   # share of the free device memory the cache may take then
    max_num_seqs: int = 64             # live requests (state slots)
    max_num_batched_tokens: int = 2048  # token budget of one step
    max_model_len: Optional[int] = None  # None = the model's max_position_embeddings
    device: int = 0
    use_graphs: bool = True            # run steps as HIP graphs, captured per shape of step
    decode_burst: int = 32             # most decode steps the device chains without the host (1: none)
    seed: int = 0

    def __post_init__(self):
        if self.dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {sorted(set(DTYPES))}, got {self.dtype!r}")
        self.dtype = DTYPES[self.dtype]
        if self.kv_block_size <= 0:
            raise ValueError("kv_block_size must be positive")
        if not (0.0 < self.cache_memory_fraction <= 1.0):
            raise ValueError("cache_memory_fraction must be in (0, 1]")
        if self.max_num_seqs <= 0 or self.max_num_batched_tokens <= 0:
            raise ValueError("max_num_seqs and max_num_batched_tokens must be positive")
