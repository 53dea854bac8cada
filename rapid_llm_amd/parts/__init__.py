"""Parts a model is assembled from.  Importing the package registers the built-in kinds."""

from . import attention, block, mlp, norm, rope  # noqa: F401  (registration)
from .base import (
    BLOCKS,
    FEED_FORWARDS,
    MIXERS,
    NORMS,
    POSITION_ENCODINGS,
    Block,
    CacheNeed,
    FeedForward,
    Mixer,
    Norm,
    ParamSpec,
    Part,
    PositionEncoding,
    Source,
)
from .runtime import Runtime

__all__ = [
    "BLOCKS",
    "FEED_FORWARDS",
    "MIXERS",
    "NORMS",
    "POSITION_ENCODINGS",
    "Block",
    "CacheNeed",
    "FeedForward",
    "Mixer",
    "Norm",
    "ParamSpec",
    "Part",
    "PositionEncoding",
    "Runtime",
    "Source",
]
