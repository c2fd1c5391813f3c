from .params import MASK64, RNG_GOLDEN, SamplingParams, advance
from .sampler import Sampler

__all__ = ["MASK64", "RNG_GOLDEN", "SamplingParams", "advance", "Sampler"]
