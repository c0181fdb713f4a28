from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, FeedForward,
                   Folded, Head, NormSink, KVNeed, LayerCache, Mixer, Norm, PAGE, PAGE_BY_8, Part, PoolNeed, PositionEncoding, StateNeed,
                   StepContext, TokenEmbedding, embedding_class, head_class, register_embedding, register_head,
                   Stream, block_class, feed_forward_class, mixer_class, norm_class,
                   position_encoding_class, register_block, register_feed_forward,
                   register_mixer, register_norm, register_position_encoding)
from . import attention, block, mlp, norm, rope  # noqa: F401  (register the built-in kinds)
from .embedding import Embedding, LMHead
from .linear import Linear
