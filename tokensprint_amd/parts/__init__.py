from tokensprint_amd.parts import attention, block, feed_forward, norm, position  # noqa: F401
from tokensprint_amd.parts.base import (
    BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, Block, BuildContext, FeedForward,
    Mixer, Norm, PagedKVNeed, Part, PositionEncoding, SlotStateNeed, TensorDecl,
    build_part, register,
)
from tokensprint_amd.parts.ends import Embedding, Head

__all__ = [
    "BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITIONS", "Block", "BuildContext",
    "FeedForward", "Mixer", "Norm", "PagedKVNeed", "Part", "PositionEncoding",
    "SlotStateNeed", "TensorDecl", "build_part", "register", "Embedding", "Head",
]
