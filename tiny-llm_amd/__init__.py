"""tiny-llm_amd: a small, whole Llama inference engine for one AMD Instinct MI355X.

Token ids in, next tokens out: typed configuration and registry, safetensors
weights, layers assembled from parts, a paged cache manager, one step function, a
scheduler, sampling, and hand-written HIP kernels for gfx950.
"""
from . import config, parts, models, weights, cache, kernels  # noqa: F401
from .config import EngineConfig, LlamaConfig
from .sampling import SamplingParams
from .engine import Engine, StepEntry

__version__ = "0.1.0"
