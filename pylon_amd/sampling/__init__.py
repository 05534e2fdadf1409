from .params import Sampling
from .rng import philox4x32, uniform
from .sampler import Sampler

__all__ = ["Sampling", "Sampler", "philox4x32", "uniform"]
