from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, CacheNeed, FragmentActs, KVNeed,
                   ParamSpec, Part, Precision, Registry, StateNeed)
from .linear import Linear
from .stream import ResidualStream
from . import norm, rope, attention, feedforward, embedding, block  # noqa: F401  (register the parts)
