from .params import SamplingParams
from .sampler import Sampler, draw_seed, splitmix64

__all__ = ["SamplingParams", "Sampler", "draw_seed", "splitmix64"]
