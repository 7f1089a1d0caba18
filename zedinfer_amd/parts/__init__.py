from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, STREAM_STEPS, Block,
                   FeedForward, HostBatch, KVCacheRequest, LayerMemory, PAGE, PageTensor, Mixer, Norm, Part, PositionEncoding, Runtime,
                   StateRequest, StepPlan, StepPlanner, StreamStep, register_block, register_embedding, register_feed_forward, register_head,
                   register_mixer, register_norm, register_position_encoding, register_stream_step)
from . import (blocks, delta_rule, embedding, feed_forward, latent_attention, linear_mixers, mixers, norms, pooled_attention,
               positions, state_space, stream_steps)  # noqa: F401  (register the kinds)
