from .base import (BLOCKS, EMBEDDINGS, EXTRAS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, SHARED, CacheNeed,
                   FragmentActs, KVNeed, ParamSpec, Part, Precision, Registry, StateNeed)
from .linear import Linear
from .stream import ResidualStream
from . import norm, rope, attention, latent, feedforward, embedding, block, mlstm, gla, composite, token_input, stream_ops, mamba2, delta, experts  # noqa: F401  (register the parts)
