from .params import GREEDY, SamplingParams
from .sampler import Sampler, SamplerRow

__all__ = ["GREEDY", "Sampler", "SamplerRow", "SamplingParams"]
