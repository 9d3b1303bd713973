"""Parts of a decoder layer, their interfaces and registries, and the generic model."""

from .registry import (ADDED_IN_PLACE, BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, Block,
                       BuildContext, DeferredNorm, PartialSums, FeedForward, Mixer, Norm, Part, PositionEncoding, register_block,
                       register_feed_forward, register_mixer, register_norm, register_position_encoding)
from .spec import LayerSpec, ModelSpec, PagedCacheSpec, ParamInfo, PartSpec, StateCacheSpec
from . import attention, block, embedding, rmsnorm, rope, swiglu  # noqa: E402,F401  (register the built-in parts)

__all__ = [
    "ADDED_IN_PLACE", "DeferredNorm", "PartialSums", "BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Block",
    "BuildContext", "FeedForward", "Mixer", "Norm", "Part", "PositionEncoding", "register_block",
    "register_feed_forward", "register_mixer", "register_norm", "register_position_encoding", "LayerSpec",
    "ModelSpec", "PagedCacheSpec", "ParamInfo", "PartSpec", "StateCacheSpec",
]
