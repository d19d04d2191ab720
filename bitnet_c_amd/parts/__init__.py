"""Parts of a layer and their registries; importing the package registers the built-in parts."""
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, CacheNeed, KVNeed, KVView,
                   LazyDelta, ParamSpec, Part, PartSpec, Registry, ResidualStream, StateNeed)
from . import attention, block, ffn, norm, position  # noqa: F401  (registration)
