"""Parts a layer is put together from.  Importing this package registers the built-in kinds."""
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, FeedForward, Mixer, Norm,
                   PagedNeed, Part, PositionEncoding, StateNeed, Stream, WeightSpec)
from . import attention, block, feedforward, norm, rotary  # noqa: F401  (registration)

__all__ = ["BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Block", "FeedForward", "Mixer",
           "Norm", "PagedNeed", "Part", "PositionEncoding", "StateNeed", "Stream", "WeightSpec"]
