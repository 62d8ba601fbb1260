"""Parts that layers are assembled from.  Importing the package registers the built-in kinds."""
from .base import (ParamSpec, KVNeed, StateNeed, CacheNeed, PartSpec, BlockSpec, LayerCall, ModelSpec,
                   Part, Norm, PositionEncoding, Mixer, FeedForward, Block, Embedding, Head, SideInput, InputShift, register, build,
                   registered, UnknownPart, two_increments, NormedIncrement, TanhIncrement)
from . import norm, position, attention, latent_attention, wide_attention, linear_attention, time_mix, state_space, mixer_sum, feed_forward, side, shift, block, ends  # noqa: F401  (registration)
