"""Parts of a layer and their registries.  Importing the package registers the
parts the framework ships."""

from . import attention, block, feedforward, norm, rope  # noqa: F401  (register themselves)
from .base import (Block, FeedForward, KVCacheView, KVNeed, Mixer, Norm, ParamSpec, Part, PositionEncoding,
                   StateNeed, StateView)
from .registry import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

__all__ = [
    "Block", "FeedForward", "KVCacheView", "KVNeed", "Mixer", "Norm", "ParamSpec", "Part", "PositionEncoding",
    "StateNeed", "StateView", "BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "LayerSpec",
    "ModelSpec", "PartSpec", "ScheduleEntry",
]
