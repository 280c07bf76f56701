from .params import SamplingParams
from .sampler import Sampler, request_seed

__all__ = ["SamplingParams", "Sampler", "request_seed"]
