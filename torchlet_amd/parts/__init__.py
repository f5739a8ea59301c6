"""Parts a layer is put together from.  Importing this package registers the built-in kinds."""
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, FeedForward, Mixer, Norm,
                   PagedNeed, Part, PositionEncoding, StateNeed, Stream, WeightSpec)
from . import attention, block, capped_attention, decayed_linear, experts, feedforward, gated_delta, latent_attention, mlstm, norm, parallel, rotary, selective_state  # noqa: F401  (registration)

__all__ = ["BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Block", "FeedForward", "Mixer",
           "Norm", "PagedNeed", "Part", "PositionEncoding", "StateNeed", "Stream", "WeightSpec"]
