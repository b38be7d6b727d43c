from . import attention, feed_forward, norm, position  # noqa: F401  (register the built-in parts)
from .base import (CacheNeed, FeedForward, Mixer, Norm, ParamSpec, Part, PositionEncoding, build_feed_forward,
                   build_mixer, build_norm, build_position, first_needed_position, register_feed_forward,
                   register_mixer, register_norm, register_position)
from .block import PreNormBlock, build_block, register_arrangement
from .model import DecoderModel

__all__ = [
    "CacheNeed", "FeedForward", "Mixer", "Norm", "ParamSpec", "Part", "PositionEncoding", "build_feed_forward",
    "build_mixer", "build_norm", "build_position", "first_needed_position", "register_feed_forward",
    "register_mixer", "register_norm", "register_position", "PreNormBlock", "build_block",
    "register_arrangement", "DecoderModel",
]
