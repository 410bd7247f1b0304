from . import (attention, block, differential_attention, embedding, input_conv, latent_attention, linear_attention, mlp, mlstm,
               norm, recurrent, rotary, routed_mlp, token_side)  # noqa: F401  (each registers its parts)
from .base import Binding, FeedForward, CacheNeed, Mixer, Norm, Part, PositionEncoding, StateNeed
from .linear import Linear

__all__ = ["Binding", "FeedForward", "CacheNeed", "Mixer", "Norm", "Part", "PositionEncoding", "StateNeed", "Linear"]
