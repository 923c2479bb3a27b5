"""Parts a model is put together from.  Importing this package registers the built-in ones."""
from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, Block, CacheSpec,
                   FeedForward, HostBatch, LayerCache, Mixer, Norm, PagedKVSpec, PageGroup, Part, PartSpec,
                   PositionEncoding, Product, StateSpec, StepState, TensorSpec)
from . import norm, rope, mlp, attention, block, embedding  # noqa: F401  (registration)
from .block import PreNormBlock, ResidualStream
from .embedding import OutputHead, TokenEmbedding
