"""Parts that layers are put together from. Importing the package registers the built-in kinds."""
from . import (attention, block, delta_rule, embedding, feed_forward, gated_block, head, hyper_connections, latent_attention, linear_attention, moe, norm,  # noqa: F401
               parallel_mixers, position, recurrent, stream_mix, talking_attention)
from .base import (AttentionMeta, Block, BuildEnv, CacheUnitView, Embedding, FeedForward, GroupView, Head, Mixer, Norm, Part,
                   PositionEncoding, StepContext, StreamMix)
from .decoder import DecoderLm
from .registry import BLOCKS, EMBEDDINGS, FAMILIES, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, STREAM_MIXES, part_class
from .spec import LayerSpec, ModelSpec, PartSpec, PlanEntry, TensorSpec

__all__ = ["AttentionMeta", "Block", "BuildEnv", "CacheUnitView", "FeedForward", "GroupView", "Head", "Mixer", "Norm", "Part",
           "PositionEncoding", "StepContext", "StreamMix", "STREAM_MIXES", "DecoderLm", "Embedding", "EMBEDDINGS", "FAMILIES", "part_class", "BLOCKS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS",
           "POSITION_ENCODINGS", "LayerSpec", "ModelSpec", "PartSpec", "PlanEntry", "TensorSpec"]
