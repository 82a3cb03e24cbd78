"""Parts of a layer and their registries; importing the package registers the built-in parts."""
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, CacheNeed, KVNeed, KVView,
                   LazyDelta, NormedDelta, ParamSpec, Part, PartSpec, Registry, ResidualStream, StateNeed)
from . import attention, block, ffn, hyper, latent, moe, norm, parallel, position, recurrent  # noqa: F401  (registration)
