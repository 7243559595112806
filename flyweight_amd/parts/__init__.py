from .base import (FeedForward, Mixer, Norm, Part, PositionEncoding, build_part, register_block,
                   register_feed_forward, register_mixer, register_norm, register_position_encoding,
                   registered)
from .linear import Linear
from . import attention, block, norm, rope, shortconv, swiglu   # noqa: F401  (registers the built-in parts)

__all__ = ["FeedForward", "Mixer", "Norm", "Part", "PositionEncoding", "Linear", "build_part",
           "register_block", "register_feed_forward", "register_mixer", "register_norm",
           "register_position_encoding", "registered"]
