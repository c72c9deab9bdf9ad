from . import attention, block, feed_forward, norm, position  # noqa: F401  (register kinds)
from .base import (CacheView, FeedForward, Mixer, Norm, PagedKVSpec, Part, PositionEncoding,
                   SlotStateSpec, StepContext, StepItem, Workspace)
from .registry import (ARRANGEMENTS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, build_part,
                       register_arrangement, register_feed_forward, register_mixer,
                       register_norm, register_position)

__all__ = [
    "ARRANGEMENTS", "CacheView", "FEED_FORWARDS", "FeedForward", "MIXERS", "Mixer", "NORMS",
    "Norm", "POSITIONS", "PagedKVSpec", "Part", "PositionEncoding", "SlotStateSpec",
    "StepContext", "StepItem", "Workspace", "build_part", "register_arrangement",
    "register_feed_forward", "register_mixer", "register_norm", "register_position",
]
