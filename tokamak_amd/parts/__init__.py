"""Parts a layer is made of.  Importing this package registers the built-in ones."""

from tokamak_amd.parts import attention, block, embedding, feed_forward, norm, rotary  # noqa: F401
from tokamak_amd.parts.base import (
    Block,
    CacheRequest,
    FeedForward,
    Mixer,
    Norm,
    Part,
    PositionEncoding,
)

__all__ = ["Block", "CacheRequest", "FeedForward", "Mixer", "Norm", "Part", "PositionEncoding"]
