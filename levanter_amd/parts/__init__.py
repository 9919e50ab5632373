"""Parts that layers are put together from. Importing the package registers the built-in kinds."""
from . import attention, block, embedding, feed_forward, head, norm, position  # noqa: F401
from .base import (AttentionMeta, Block, BuildEnv, CacheUnitView, Embedding, FeedForward, GroupView, Head, Mixer, Norm, Part,
                   PositionEncoding, StepContext)
from .decoder import DecoderLm
from .registry import BLOCKS, EMBEDDINGS, FAMILIES, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, part_class
from .spec import LayerSpec, ModelSpec, PartSpec, PlanEntry, TensorSpec

__all__ = ["AttentionMeta", "Block", "BuildEnv", "CacheUnitView", "FeedForward", "GroupView", "Head", "Mixer", "Norm", "Part",
           "PositionEncoding", "StepContext", "DecoderLm", "Embedding", "EMBEDDINGS", "FAMILIES", "part_class", "BLOCKS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS",
           "POSITION_ENCODINGS", "LayerSpec", "ModelSpec", "PartSpec", "PlanEntry", "TensorSpec"]
