from tokensprint_amd.parts import (attention, block, feed_forward, latent_attention, mamba2,  # noqa: F401
                                   norm, position, recurrent)
from tokensprint_amd.parts.base import (
    BLOCKS, EMBEDDINGS, FEED_FORWARDS, FILTERS, HEADS, MIXERS, NORMS, POSITIONS, Block,
    BuildContext, FeedForward, Mixer, Norm, OutputHead, PagedKVNeed, PagedLatentNeed, Part,
    PositionEncoding, SlotStateNeed, StreamFilter, TensorDecl, TokenEmbedding, build_part, register,
)
from tokensprint_amd.parts.ends import Embedding, Head

__all__ = [
    "BLOCKS", "EMBEDDINGS", "FILTERS", "PagedLatentNeed", "StreamFilter", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITIONS", "Block",
    "BuildContext", "FeedForward", "Mixer", "Norm", "OutputHead", "PagedKVNeed", "Part",
    "PositionEncoding", "SlotStateNeed", "TensorDecl", "TokenEmbedding", "build_part",
    "register", "Embedding", "Head",
]
