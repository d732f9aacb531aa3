from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, Block, CacheNeed,
                   FeedForward, Mixer, Norm, Part, PositionEncoding, Stream, register_block,
                   register_embedding, register_feed_forward, register_head, register_mixer,
                   register_norm, register_position)
from .spec import LayerCall, LayerSpec, ModelSpec, ParamDecl, PartSpec
from . import block, embedding, feed_forward, mixer, norm, position  # noqa: F401  (register the built-in parts)
