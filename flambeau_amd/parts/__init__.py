"""Parts a model is put together from.  Importing this package registers the built-in ones."""
from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, BiasedProduct, Block, CacheSpec,
                   FeedForward, HostBatch, JoinedCacheSpec, LayerCache, Mixer, Norm, PagedKVSpec, PagedRowSpec, PageGroup, Part, PartSpec,
                   PositionEncoding, Product, StateSpec, StepState, TensorSpec)
from . import norm, rope, mlp, attention, block, embedding, latent_attention, mlstm, moe, linear_recurrence, side_by_side  # noqa: F401  (registration)
from .block import ParallelBlock, PreNormBlock, ResidualStream, StreamReentry
from .embedding import OutputHead, TokenEmbedding
