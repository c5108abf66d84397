from . import attention, block, embedding, feedforward, norm, rope  # noqa: F401
from .base import (
    ARRANGEMENTS,
    EMBEDDINGS,
    FEED_FORWARDS,
    HEADS,
    MIXERS,
    NORMS,
    POSITIONS,
    Arrangement,
    BuildContext,
    Embedding,
    FeedForward,
    Head,
    Mixer,
    Norm,
    PagedKVNeed,
    PagedNeed,
    ParamDecl,
    Part,
    PositionEncoding,
    RotaryPositionEncoding,
    RunBinding,
    StateNeed,
    register_arrangement,
)
from .decoder import Decoder

__all__ = [
    "ARRANGEMENTS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITIONS",
    "Arrangement", "BuildContext", "Decoder", "Embedding", "FeedForward", "Head", "Mixer", "Norm",
    "PagedKVNeed", "PagedNeed", "ParamDecl", "Part", "PositionEncoding", "RotaryPositionEncoding", "RunBinding", "StateNeed",
    "register_arrangement",
]
