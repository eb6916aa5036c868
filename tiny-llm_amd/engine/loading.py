"""From a model folder (or a configuration and a seed) to a decoder with its cache
and a runner: the one way every front end (generation, replay, bench) builds a model."""
from __future__ import annotations

from typing import Mapping, Optional

import torch

from ..cache import CacheManager
from ..config import EngineConfig, resolve, read_config_json
from ..kernels import library
from ..models.decoder import Decoder
from ..weights import init_random_weights, load_weights
from .step import ModelRunner


class NoDevice(RuntimeError):
    pass


def require_gpu(device: int = 0) -> torch.device:
    if not torch.cuda.is_available():
        raise NoDevice("no GPU is visible; this engine has no CPU path")
    library.load()
    torch.cuda.set_device(device)
    return torch.device(f"cuda:{device}")


def build_decoder(config: Mapping, dtype: str, device) -> tuple:
    cfg, spec = resolve(config)
    return cfg, Decoder(spec, dtype=dtype, device=device)


def load_model(model_path: str, engine: EngineConfig):
    """config.json chooses the model class; weights come from the folder's safetensors."""
    device = require_gpu(engine.device)
    cfg, dec = build_decoder(read_config_json(model_path), engine.dtype, device)
    load_weights(dec, model_path)
    return cfg, dec


def random_model(config: Mapping, engine: EngineConfig, seed: int = 0, std: Optional[float] = None,
                 norm_std: float = 0.0):
    """A decoder with seeded random weights made on the device (no files)."""
    device = require_gpu(engine.device)
    cfg, dec = build_decoder(config, engine.dtype, device)
    init_random_weights(dec, seed, float(config.get("initializer_range", 0.02)) if std is None else std, norm_std)
    return cfg, dec


def plan_cache_blocks(engine: EngineConfig, max_len: int, bytes_per_block: int, free_bytes: Optional[int]) -> int:
    """How many cache blocks every group gets.  A number in the configuration is taken as it is
    (`num_kv_blocks`, or `max_cache_tokens` in blocks).  Otherwise: the worst case of
    `max_num_seqs` requests of `max_len` tokens, which can never run out (the reference's rule,
    tiny_llm/runtime/cuda/cuda_runtime.cpp:510-515), capped by `cache_memory_fraction` of the
    device memory that is free once the weights are resident; a smaller pool is what the
    scheduler's preemption is for."""
    bs = engine.kv_block_size
    if engine.num_kv_blocks is not None:
        return max(1, int(engine.num_kv_blocks))
    if engine.max_cache_tokens is not None:
        return max(1, -(-engine.max_cache_tokens // bs))
    blocks = engine.max_num_seqs * (-(-max_len // bs))
    if free_bytes is not None and bytes_per_block > 0:
        fit = int(free_bytes * engine.cache_memory_fraction) // bytes_per_block
        if fit < 1:
            raise MemoryError(f"no device memory for the cache: one block of {bs} tokens takes "
                              f"{bytes_per_block} bytes, {free_bytes} bytes are free")
        blocks = min(blocks, fit)
    return max(1, blocks)


def build_runner(dec: Decoder, engine: EngineConfig) -> ModelRunner:
    max_len = engine.max_model_len or dec.spec.max_position
    max_len = min(max_len, dec.spec.max_position)
    bs = engine.kv_block_size
    cache_specs, state_specs = dec.cache_specs(), dec.state_specs()
    elt = torch.empty((), dtype=dec.dtype).element_size()
    per_block = CacheManager(cache_specs, state_specs, bs, 1, 1).elements_per_block() * elt
    free = torch.cuda.mem_get_info(dec.device)[0] if dec.device.type == "cuda" else None
    blocks = plan_cache_blocks(engine, max_len, per_block, free)
    cache = CacheManager(cache_specs, state_specs, bs, blocks, engine.max_num_seqs)
    cache.allocate_tensors(dec.dtype, dec.device)
    return ModelRunner(dec, cache, engine.max_num_batched_tokens, max_len)
