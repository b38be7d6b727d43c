from . import attention, embedding, feed_forward, norm, position  # noqa: F401  (register the built-in parts)
from .base import (CacheNeed, Embedding, FeedForward, Mixer, Norm, OutputHead, ParamSpec, Part, PositionEncoding,
                   build_embedding, build_feed_forward, build_head, register_embedding, register_head,
                   build_mixer, build_norm, build_position, first_needed_position, register_feed_forward, register_retention,
                   register_mixer, register_norm, register_position)
from .block import PreNormBlock, build_block, register_arrangement
from .model import DecoderModel

__all__ = [
    "CacheNeed", "Embedding", "OutputHead", "build_embedding", "build_head", "register_embedding", "register_head",
    "FeedForward", "Mixer", "Norm", "ParamSpec", "Part", "PositionEncoding", "build_feed_forward",
    "build_mixer", "build_norm", "build_position", "first_needed_position", "register_feed_forward", "register_retention",
    "register_mixer", "register_norm", "register_position", "PreNormBlock", "build_block",
    "register_arrangement", "DecoderModel",
]
