"""Parts: importing the package registers the built-in kinds."""

from . import attention, block, embedding, mlp, rmsnorm, rotary  # noqa: F401
from .base import (  # noqa: F401
    BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, Block, CacheNeed,
    Embedding, FeedForward, Head, Mixer, Norm, ParamSource, ParamSpec, Part, PartSpec, PositionEncoding,
    RotaryTables, RunLimits, Runtime, StateNeed, register_block, register_embedding,
    register_feed_forward, register_head, register_mixer, register_norm, register_position_encoding,
)
