"""Parts that layers are assembled from.  Importing the package registers the built-in kinds."""
from .base import (ParamSpec, KVNeed, StateNeed, CacheNeed, PartSpec, BlockSpec, LayerCall, ModelSpec,
                   Part, Norm, PositionEncoding, Mixer, FeedForward, Block, Embedding, Head, register, build, registered,
                   UnknownPart, two_increments)
from . import norm, position, attention, feed_forward, block, ends  # noqa: F401  (registration)
