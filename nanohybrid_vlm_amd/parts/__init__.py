"""Parts of a model: mixers, feed-forwards, norms, position encodings, blocks.
Importing the package registers the built-in ones."""
from . import blocks, feed_forward, mixers, norms, positions  # noqa: F401  (registration)
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, CacheView, PagedKVNeed, ParamSpec, Part,
                   StateNeed)

__all__ = ["BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "CacheView", "PagedKVNeed", "ParamSpec",
           "Part", "StateNeed"]
