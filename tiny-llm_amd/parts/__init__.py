from .base import (Part, Embedding, Head, Norm, Mixer, FeedForward, PositionEncoding, Block, ChannelScale, StreamPart, WeightSpec, CacheSpec,
                   CacheTensor, StateSpec, LayerCache, add_to_residual, project_into_residual, EMBEDDINGS, HEADS,
                   NORMS, MIXERS, FEED_FORWARDS, POSITION_ENCODINGS, SCALES, STREAM_PARTS, BLOCKS, REGISTRIES, register_embedding,
                   register_head, register_norm, register_mixer, register_feed_forward,
                   register_position_encoding, register_scale, register_stream_part, register_block)
from . import norm, rotary, attention, latent_attention, delta_rule, time_mix, parallel, mlp, moe, block, embedding, stream  # noqa: F401  (fills the registries)
