from .params import SamplingParams
from .sampler import SAMPLER_EPS, Sampler

__all__ = ["SamplingParams", "Sampler", "SAMPLER_EPS"]
