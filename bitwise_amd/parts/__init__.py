"""Parts a model is assembled from.  Importing the package registers the built-in parts."""

from . import attention, block, embedding, mlp, norm, rope  # noqa: F401  (registration side effects)
from .base import (  # noqa: F401
    Block, CacheSpec, Embedding, FeedForward, Head, LayerCall, LayerSpec, Mixer, ModelSpec, Norm, Part, PartSpec, PositionEncoding,
    StateSpec, TensorSpec, register_block, register_feed_forward, register_mixer, register_norm,
    register_position_encoding, register_embedding, register_head,
)
