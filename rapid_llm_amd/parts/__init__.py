"""Parts a model is assembled from.  Importing the package registers the built-in kinds."""

from . import attention, block, embedding, mlp, norm, rope  # noqa: F401  (registration)
from .base import (
    BLOCKS,
    EMBEDDINGS,
    FEED_FORWARDS,
    MIXERS,
    NORMS,
    OUTPUT_PROJECTIONS,
    POSITION_ENCODINGS,
    Block,
    CacheNeed,
    Embedding,
    FeedForward,
    Mixer,
    Norm,
    OutputProjection,
    ParamSpec,
    Part,
    PositionEncoding,
    Source,
    StateSpec,
)
from .runtime import Runtime

__all__ = [
    "BLOCKS",
    "EMBEDDINGS",
    "FEED_FORWARDS",
    "MIXERS",
    "NORMS",
    "OUTPUT_PROJECTIONS",
    "POSITION_ENCODINGS",
    "Block",
    "CacheNeed",
    "Embedding",
    "FeedForward",
    "Mixer",
    "Norm",
    "OutputProjection",
    "ParamSpec",
    "Part",
    "PositionEncoding",
    "Runtime",
    "Source",
    "StateSpec",
]
