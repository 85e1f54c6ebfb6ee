"""Parts that models are put together from; importing this registers the built-in kinds."""

from . import attention, block, embedding, feed_forward, head, norms, positions  # noqa: F401
from .base import (
    BLOCKS,
    EMBEDDINGS,
    FEED_FORWARDS,
    HEADS,
    MIXERS,
    NORMS,
    POSITION_ENCODINGS,
    Block,
    FeedForward,
    Mixer,
    Norm,
    Part,
    PositionEncoding,
    TensorSpec,
    build_part,
    register_block,
    register_embedding,
    register_feed_forward,
    register_head,
    register_mixer,
    register_norm,
    register_position_encoding,
)
from .model import DecoderModel

__all__ = [
    "Part", "Norm", "Mixer", "FeedForward", "PositionEncoding", "Block", "TensorSpec",
    "DecoderModel", "build_part",
    "NORMS", "MIXERS", "FEED_FORWARDS", "POSITION_ENCODINGS", "BLOCKS", "EMBEDDINGS", "HEADS",
    "register_norm", "register_mixer", "register_feed_forward", "register_position_encoding",
    "register_block", "register_embedding", "register_head",
]
