from .params import SamplingParams
from .sampler import Sampler, uniform_draw

__all__ = ["SamplingParams", "Sampler", "uniform_draw"]
