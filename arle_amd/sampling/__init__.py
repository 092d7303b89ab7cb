from .params import SamplingParams
from .sampler import Sampler, uniform

__all__ = ["SamplingParams", "Sampler", "uniform"]
