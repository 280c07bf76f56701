"""Parts that blocks are put together from; importing this package registers the built-in ones."""
from .base import Block, FeedForward, Mixer, Norm, PagedKVNeed, ParamSpec, Part, PositionEncoding, StateNeed
from . import attention, block, embedding, ffn, norm, rope  # noqa: F401  (registration)

__all__ = ["Block", "FeedForward", "Mixer", "Norm", "PagedKVNeed", "ParamSpec", "Part", "PositionEncoding",
           "StateNeed"]
