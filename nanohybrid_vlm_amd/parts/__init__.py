"""Parts of a model: mixers, feed-forwards, norms, position encodings, blocks, embeddings.
Importing the package registers the built-in ones."""
from . import blocks, embeddings, feed_forward, latent, mixers, norms, positions  # noqa: F401  (registration)
from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, CacheView, CombinedNeed, PagedKVNeed, ParamSpec,
                   Part, StateNeed)

__all__ = ["BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "CacheView", "CombinedNeed", "PagedKVNeed", "ParamSpec",
           "Part", "StateNeed"]
