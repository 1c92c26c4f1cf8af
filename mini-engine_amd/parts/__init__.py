"""Parts of a decoder layer. Importing this package registers the built-in kinds."""

from . import attention, mlp, norm, rotary  # noqa: F401
from .base import (
    BLOCK_ARRANGEMENTS,
    FEED_FORWARDS,
    MIXERS,
    NORMS,
    POSITION_ENCODINGS,
    FeedForward,
    KVBinding,
    KVCacheNeed,
    Mixer,
    Norm,
    PositionEncoding,
    StateBinding,
    StateNeed,
)
from .block import PreNormBlock, build_block
from .decoder import Decoder

__all__ = [
    "BLOCK_ARRANGEMENTS",
    "Decoder",
    "FEED_FORWARDS",
    "FeedForward",
    "KVBinding",
    "KVCacheNeed",
    "MIXERS",
    "Mixer",
    "NORMS",
    "Norm",
    "POSITION_ENCODINGS",
    "PositionEncoding",
    "PreNormBlock",
    "StateBinding",
    "StateNeed",
    "build_block",
]
