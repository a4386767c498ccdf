from . import attention, block, embedding, mlp, norm, rotary  # noqa: F401  (each registers its parts)
from .base import Binding, FeedForward, CacheNeed, Mixer, Norm, Part, PositionEncoding, StateNeed
from .linear import Linear

__all__ = ["Binding", "FeedForward", "CacheNeed", "Mixer", "Norm", "Part", "PositionEncoding", "StateNeed", "Linear"]
