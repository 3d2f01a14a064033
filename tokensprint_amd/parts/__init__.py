from tokensprint_amd.parts import attention, block, feed_forward, norm, position  # noqa: F401
from tokensprint_amd.parts.base import (
    BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, Block, BuildContext,
    FeedForward, Mixer, Norm, OutputHead, PagedKVNeed, Part, PositionEncoding, SlotStateNeed,
    TensorDecl, TokenEmbedding, build_part, register,
)
from tokensprint_amd.parts.ends import Embedding, Head

__all__ = [
    "BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITIONS", "Block",
    "BuildContext", "FeedForward", "Mixer", "Norm", "OutputHead", "PagedKVNeed", "Part",
    "PositionEncoding", "SlotStateNeed", "TensorDecl", "TokenEmbedding", "build_part",
    "register", "Embedding", "Head",
]
