from . import (attention, block, connection, differential_attention, embedding, feed_forward,  # noqa: F401
               latent_attention, linear_attention, norm, position, side_by_side,  # noqa: F401
               state_space)  # noqa: F401  (register kinds)
from .base import (CacheView, Embedding, FeedForward, Head, Mixer, Norm, PagedKVSpec, Part,
                   PositionEncoding, SlotStateSpec, StepContext, StepItem, Workspace)
from .registry import (ARRANGEMENTS, CONNECTIONS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, ROLES,
                       build_part, register_arrangement, register_embedding, register_feed_forward,
                       register_connection, register_head, register_mixer, register_norm, register_position)

__all__ = [
    "ARRANGEMENTS", "CONNECTIONS", "CacheView", "EMBEDDINGS", "Embedding", "FEED_FORWARDS", "FeedForward", "HEADS",
    "Head", "MIXERS", "Mixer", "NORMS", "Norm", "POSITIONS", "PagedKVSpec", "Part",
    "PositionEncoding", "ROLES", "SlotStateSpec", "StepContext", "StepItem", "Workspace",
    "build_part", "register_arrangement", "register_embedding", "register_feed_forward",
    "register_connection",
    "register_head", "register_mixer", "register_norm", "register_position",
]
