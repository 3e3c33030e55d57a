from .sampler import Sampler, splitmix64, uniform

__all__ = ["Sampler", "splitmix64", "uniform"]
