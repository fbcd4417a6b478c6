from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, Block,
                   FeedForward, HostBatch, KVCacheRequest, LayerMemory, PAGE, PageTensor, Mixer, Norm, Part, PositionEncoding, Runtime,
                   StateRequest, StepPlan, StepPlanner, register_block, register_embedding, register_feed_forward, register_head,
                   register_mixer, register_norm, register_position_encoding)
from . import blocks, embedding, feed_forward, mixers, norms, positions  # noqa: F401  (register the kinds)
