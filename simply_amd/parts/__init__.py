"""Parts that blocks are put together from; importing this package registers the built-in ones."""
from .base import (Block, CompositeNeed, FeedForward, Mixer, Norm, PagedKVNeed, ParamSpec, Part,
                   PositionEncoding, StateNeed, StreamPart)
from . import attention, block, embedding, ffn, gated_attention, latent, linear_state, norm, parallel, recurrent, rope, side  # noqa: F401  (registration)

__all__ = ["Block", "CompositeNeed", "FeedForward", "Mixer", "Norm", "PagedKVNeed", "ParamSpec", "Part",
           "PositionEncoding", "StateNeed", "StreamPart"]
