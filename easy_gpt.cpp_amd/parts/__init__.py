from . import (attention, block, branch_mixers, depth_average, embedding, expert_mixture, feed_forward, gated_recurrence,  # noqa: F401
               head_attention, local_attention, norm, position, recurrent_mixers)      # (register the built-in parts)
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
    StreamJoin,
    make_part,
    register_part,
)
from .model import CacheGroup, Model, build_model
from .spec import LayerSpec, ModelSpec, ParamSpec, PartSpec, RunSpec

__all__ = [
    "BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Block", "CacheGroup", "CacheNeed",
    "CacheView", "Embedding", "FeedForward", "LayerSpec", "Mixer", "Model", "ModelSpec", "Norm", "OutputHead", "PagedTensor", "ParamSpec", "Part",
    "PartSpec", "PendingNorm", "PositionEncoding", "RunSpec", "StateNeed", "StateView", "StreamJoin", "build_model", "make_part",
    "register_part",
]
