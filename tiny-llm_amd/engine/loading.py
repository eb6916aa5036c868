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


def build_runner(dec: Decoder, engine: EngineConfig) -> ModelRunner:
    max_len = engine.max_model_len or dec.spec.max_position
    max_len = min(max_len, dec.spec.max_position)
    bs = engine.kv_block_size
    if engine.num_kv_blocks is not None:
        blocks = engine.num_kv_blocks
    elif engine.max_cache_tokens is not None:
        blocks = -(-engine.max_cache_tokens // bs)
    else:
        blocks = engine.max_num_seqs * (-(-max_len // bs))
    cache = CacheManager(dec.cache_specs(), dec.state_specs(), bs, max(1, blocks), engine.max_num_seqs)
    cache.allocate_tensors(dec.dtype, dec.device)
    return ModelRunner(dec, cache, engine.max_num_batched_tokens, max_len)
