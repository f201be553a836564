"""Parts a layer is made of.  Importing this package registers the built-in ones."""

from tokamak_amd.parts import (attention, block, embedding, feed_forward, latent_attention, linear_attention, norm,  # noqa: F401
                               pooled_attention, rotary, routed_experts, scale, state_space, time_mix)
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
