from .base import (
    BLOCKS,
    EMBEDDINGS,
    FEED_FORWARDS,
    HEADS,
    MIXERS,
    NORMS,
    POSITIONS,
    Block,
    Embedding,
    FeedForward,
    Head,
    KVNeed,
    Mixer,
    Norm,
    ParamSpec,
    Part,
    PositionEncoding,
    StateNeed,
)
from .model import Model

__all__ = [
    "BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITIONS",
    "Block", "Embedding", "FeedForward", "Head", "KVNeed", "Mixer", "Model", "Norm",
    "ParamSpec", "Part", "PositionEncoding", "StateNeed",
]
