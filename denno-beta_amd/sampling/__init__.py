from .params import SamplingParams
from .rng import entropy_seed, uniform
from .sampler import Sampler

__all__ = ["SamplingParams", "Sampler", "entropy_seed", "uniform"]
