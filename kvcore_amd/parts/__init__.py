"""Parts: importing the package registers the built-in kinds."""

from . import attention, block, embedding, mlp, rmsnorm, rotary  # noqa: F401
from .base import (  # noqa: F401
    BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, CacheNeed, FeedForward, Mixer,
    Norm, ParamSource, ParamSpec, Part, PartSpec, PositionEncoding, RotaryTables, Runtime, StateNeed,
    register_block, register_feed_forward, register_mixer, register_norm, register_position_encoding,
)
