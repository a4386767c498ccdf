from .sampler import Sampler, splitmix64, uniform01

__all__ = ["Sampler", "splitmix64", "uniform01"]
