from . import attention, block, embedding, feed_forward, norm, position  # noqa: F401  (register the built-in parts)
from .base import (
    BLOCKS,
    FEED_FORWARDS,
    MIXERS,
    NORMS,
    POSITION_ENCODINGS,
    Block,
    CacheNeed,
    CacheView,
    Embedding,
    FeedForward,
    Mixer,
    Norm,
    OutputHead,
    PagedTensor,
    Part,
    PendingNorm,
    PositionEncoding,
    StateNeed,
    StateView,
    make_part,
    register_part,
)
from .model import CacheGroup, Model, build_model
from .spec import LayerSpec, ModelSpec, ParamSpec, PartSpec, RunSpec

__all__ = [
    "BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Block", "CacheGroup", "CacheNeed",
    "CacheView", "Embedding", "FeedForward", "LayerSpec", "Mixer", "Model", "ModelSpec", "Norm", "OutputHead", "PagedTensor", "ParamSpec", "Part",
    "PartSpec", "PendingNorm", "PositionEncoding", "RunSpec", "StateNeed", "StateView", "build_model", "make_part",
    "register_part",
]
