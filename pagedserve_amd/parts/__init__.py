from . import attention, block, embedding, feed_forward, norm, position  # noqa: F401  (register kinds)
from .base import (CacheView, Embedding, FeedForward, Head, Mixer, Norm, PagedKVSpec, Part,
                   PositionEncoding, SlotStateSpec, StepContext, StepItem, Workspace)
from .registry import (ARRANGEMENTS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, ROLES,
                       build_part, register_arrangement, register_embedding, register_feed_forward,
                       register_head, register_mixer, register_norm, register_position)

__all__ = [
    "ARRANGEMENTS", "CacheView", "EMBEDDINGS", "Embedding", "FEED_FORWARDS", "FeedForward", "HEADS",
    "Head", "MIXERS", "Mixer", "NORMS", "Norm", "POSITIONS", "PagedKVSpec", "Part",
    "PositionEncoding", "ROLES", "SlotStateSpec", "StepContext", "StepItem", "Workspace",
    "build_part", "register_arrangement", "register_embedding", "register_feed_forward",
    "register_head", "register_mixer", "register_norm", "register_position",
]
