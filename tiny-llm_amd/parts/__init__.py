from .base import (Part, Norm, Mixer, FeedForward, PositionEncoding, Block, WeightSpec, CacheSpec, StateSpec,
                   LayerCache, add_to_residual, NORMS, MIXERS, FEED_FORWARDS, POSITION_ENCODINGS, BLOCKS,
                   register_norm, register_mixer, register_feed_forward, register_position_encoding,
                   register_block)
from . import norm, rotary, attention, mlp, block, embedding  # noqa: F401  (fills the registries)
