from .base import (Part, Embedding, Head, Norm, Mixer, FeedForward, PositionEncoding, Block, WeightSpec, CacheSpec,
                   CacheTensor, StateSpec, LayerCache, add_to_residual, project_into_residual, EMBEDDINGS, HEADS,
                   NORMS, MIXERS, FEED_FORWARDS, POSITION_ENCODINGS, BLOCKS, REGISTRIES, register_embedding,
                   register_head, register_norm, register_mixer, register_feed_forward,
                   register_position_encoding, register_block)
from . import norm, rotary, attention, mlp, block, embedding  # noqa: F401  (fills the registries)
