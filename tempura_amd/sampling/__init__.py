from .params import SamplingParams
from .sampler import Sampler, TokenLogprob, uniform_draw

__all__ = ["SamplingParams", "Sampler", "TokenLogprob", "uniform_draw"]
