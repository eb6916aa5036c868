"""From a model folder (or a configuration and a seed) to a decoder with its cache
and a runner: the one way every front end (generation, replay, bench) builds a model."""
from __future__ import annotations

from typing import Mapping, Optional, Sequence

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


def plan_cache_blocks(engine: EngineConfig, max_len: int, bytes_per_block, free_bytes: Optional[int],
                      held_at_most: Optional[Sequence[int]] = None):
    """How many cache blocks each group's pool gets.

    bytes_per_block: one number per cache group (a single number: one group; an int is returned
    then).  held_at_most: per group the blocks ONE request of `max_len` tokens holds at most (a full
    group ceil(max_len / block), a window group its window and a step's token budget); None: every
    group is full.

    A number in the configuration (`num_kv_blocks`, or `max_cache_tokens` in blocks) is what a
    full group gets; a group that never holds that much gets its own worst case instead.
    Otherwise every group gets the worst case of `max_num_seqs` requests, which can never run out
    (the reference's rule, tiny_llm/runtime/cuda/cuda_runtime.cpp:510-515); if that is more than
    `cache_memory_fraction` of the device memory that is free once the weights are resident, all
    groups shrink by one factor (each still serves the same number of longest requests); a smaller
    pool is what the scheduler's preemption is for."""
    bs = engine.kv_block_size
    single = not isinstance(bytes_per_block, (list, tuple))
    per_block = [int(bytes_per_block)] if single else [int(b) for b in bytes_per_block]
    whole = -(-max_len // bs)
    held = [whole] * len(per_block) if held_at_most is None else [max(1, int(h)) for h in held_at_most]
    worst = [engine.max_num_seqs * h for h in held]
    if engine.num_kv_blocks is not None or engine.max_cache_tokens is not None:
        given = int(engine.num_kv_blocks) if engine.num_kv_blocks is not None else -(-engine.max_cache_tokens // bs)
        blocks = [max(1, given if h >= whole else min(given, w)) for h, w in zip(held, worst)]
    else:
        blocks = list(worst)
        need = sum(n * b for n, b in zip(blocks, per_block))
        if free_bytes is not None and need > 0:
            room = int(free_bytes * engine.cache_memory_fraction)
            if room < sum(per_block):
                raise MemoryError(f"no device memory for the cache: one block of {bs} tokens per group takes "
                                  f"{sum(per_block)} bytes, {free_bytes} bytes are free")
            if need > room:
                blocks = [max(1, n * room // need) for n in blocks]
    return blocks[0] if single else blocks


def build_runner(dec: Decoder, engine: EngineConfig) -> ModelRunner:
    max_len = engine.max_model_len or dec.spec.max_position
    max_len = min(max_len, dec.spec.max_position)
    bs = engine.kv_block_size
    cache_specs, state_specs = dec.cache_specs(), dec.state_specs()
    elt = torch.empty((), dtype=dec.dtype).element_size()
    probe = CacheManager(cache_specs, state_specs, bs, 1, 1)
    per_block = [n * elt for n in probe.elements_per_block()]
    free = torch.cuda.mem_get_info(dec.device)[0] if dec.device.type == "cuda" else None
    held = probe.blocks_held_at_most(max_len, engine.max_num_batched_tokens)
    blocks = plan_cache_blocks(engine, max_len, per_block, free, held)
    cache = CacheManager(cache_specs, state_specs, bs, blocks, engine.max_num_seqs)
    cache.allocate_tensors(dec.dtype, dec.device)
    return ModelRunner(dec, cache, engine.max_num_batched_tokens, max_len)
