"""Parts of a layer and their registries.  Importing the package registers the
parts the framework ships."""

from . import attention, block, embedding, feedforward, norm, rope  # noqa: F401  (register themselves)
from .base import (Block, Embedding, FeedForward, Head, KVCacheView, KVNeed, Mixer, Norm, ParamSpec, Part,
                   PositionEncoding, StateNeed, StateView)
from .registry import BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

__all__ = [
    "Block", "Embedding", "FeedForward", "Head", "KVCacheView", "KVNeed", "Mixer", "Norm", "ParamSpec", "Part",
    "PositionEncoding", "StateNeed", "StateView", "BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS",
    "POSITION_ENCODINGS", "LayerSpec", "ModelSpec", "PartSpec", "ScheduleEntry",
]
